/*
 * spiral_mi355.h - C ABI of libspiral_mi355.so, the MI355X (gfx950) implementation of the
 * data-parallel hot path of mrakgr/Spiral-s-ML-Library: tiled GEMM C = A.B^T, dense-layer
 * forward, and the row primitives (reductions, scans, softmax, argmax, categorical sampling).
 *
 * The reference has no C ABI: its device entry points are `extern "C" __global__ entry{N}`
 * kernels compiled at import time by CuPy's RawModule and launched with
 * `fn((blocks,),(threads,),(arrays...),shared_mem=S)` (corecuda/base.spi:52-111), with all
 * shapes baked in as compile-time literals.  Each function below names the reference
 * interface it stands in for.
 *
 * Conventions (all functions):
 *   - every tensor is row-major, contiguous, innermost stride 1 (corebase/tensorm/utils.spir:27);
 *   - device pointers must be 16-byte aligned (corecuda/base.spi:158 asserts the same);
 *   - the library borrows the buffers, writes results in place, never allocates device memory
 *     and never synchronises: work is enqueued on `stream` (a hipStream_t, NULL = default stream);
 *   - return value: SP_OK (0) or a negative sp_status; sp_last_error_string() describes the
 *     last failure on the calling thread.  Nothing throws.
 */
#ifndef SPIRAL_MI355_H
#define SPIRAL_MI355_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    SP_OK = 0,
    SP_ERR_NULL = -1,        /* a required pointer is NULL */
    SP_ERR_SHAPE = -2,       /* a dimension is non-positive, too large, or violates a divisibility rule */
    SP_ERR_ALIGN = -3,       /* a pointer is not 16-byte aligned */
    SP_ERR_DTYPE = -4,       /* unsupported dtype combination */
    SP_ERR_ARG = -5,         /* any other invalid argument (alpha == 0, unknown op, bad mask size ...) */
    SP_ERR_UNSUPPORTED = -6, /* valid request this build has no kernel for */
    SP_ERR_DEVICE = -7       /* HIP reported an error at launch; see sp_last_error_string() */
} sp_status;

typedef enum { SP_F32 = 0, SP_F16 = 1, SP_BF16 = 2 } sp_dtype;

/* ------------------------------------------------------------------------------------------ */
/* library                                                                                     */
/* ------------------------------------------------------------------------------------------ */

/* Human-readable description of the last error on this thread ("" if none). */
const char* sp_last_error_string(void);

typedef struct {
    char name[128];
    char arch[64];              /* gcnArchName, must start with "gfx950" for the kernels to run */
    int32_t compute_units;
    int32_t wavefront_size;
    int32_t lds_bytes_per_cu;   /* shared memory per workgroup limit */
    int32_t max_clock_khz;
    int64_t hbm_bytes;
    int32_t l2_bytes;
} sp_device_info_t;

/* Replaces the host-side device probing of corecuda/base.spi:73 (SM-count assert) and
 * ml/max_blocks_per_sm.py:2-31 (device attribute queries). */
int sp_device_info(sp_device_info_t* out);

/* Occupancy report for a named kernel of this library: "gemm_bf16_256x256_4w", "gemm_f16_256x256_4w"
 * (four-wave kernel of the large 16-bit shapes), "gemm_bf16_256x256", "gemm_f16_256x256",
 * "gemm_bf16_128x128", "gemm_f32_64x64", "row_ops", "row_ops_scalars" (sp_row_ops without probs/cdf
 * outputs), "row_map", "mlp_forward", "mlp_forward_wide".
 * Registers, static LDS bytes and resident workgroups per CU (dynamic LDS not included).  Stands in
 * for ml/max_blocks_per_sm.py:2-31.  Returns SP_ERR_ARG for an unknown name. */
typedef struct {
    int32_t vgprs;              /* architected + accumulation VGPRs per lane (from the code object) */
    int32_t sgprs;
    int32_t static_lds_bytes;
    int32_t threads_per_block;
    int32_t max_blocks_per_cu;
} sp_kernel_info_t;
int sp_kernel_info(const char* kernel_family, sp_kernel_info_t* out);

/* Measurement aid: `out` (device memory, 32768 slots of two 64-bit words = 512 KiB, zeroed by the caller) receives,
 * in the slot of every SIMD a workgroup of the sampling kernel ran on (slot = XCD number * 4096 + bits 15:4 of the
 * hardware id: shader engine, shader array, compute unit, SIMD), that unit's cycle counter and the constant 100 MHz
 * counter, read at the point of `stream` where the call is enqueued; slots of places the kernel did not reach stay
 * zero.  Two samples around a stretch of work give the clock the compute units ran at during it: per slot filled in
 * both, (cycles1 - cycles0) / (ticks1 - ticks0) * 100 MHz (every unit's cycle counter runs from a start of its own,
 * so samples are only compared slot by slot).  Power-limited kernels run well below the nominal 2.4 GHz.  Stands
 * beside the host-side device probing of corecuda/base.spi:73; the reference has no counterpart. */
int sp_clock_sample(uint64_t* out, void* stream);

/* ------------------------------------------------------------------------------------------ */
/* GEMM                                                                                        */
/* ------------------------------------------------------------------------------------------ */

#define SP_GEMM_RELU 0x1u       /* apply max(0, .) after bias (build extension; the reference
                                   fuses nothing: game/leduc/model_cem.spi:59 "TODO: Fuse this relu") */
#define SP_GEMM_FORCE_GENERIC 0x100u /* testing aid: use the shape-agnostic kernel even for tileable shapes */

/*
 * C = alpha * A . B^T + beta * C  [+ bias[n]] [ReLU]
 *
 * Replaces `matmul_tf32 false true alpha a b beta c` (ml/matmul/run.spi:21-26 ->
 * matmul_tf32_template, ml/matmul/kernel.spi:25-240; generated entry point
 * `entry0(float* A, float* B, float* C)`, ml/matmul/run.py:300,1232) and the grid-strided
 * variant tests/matmul/test3_kernel.spi:148.
 *
 *   A (M,K), B (N,K), C (M,N) row-major.  dtype_in in {SP_F32, SP_F16, SP_BF16} is the storage
 *   type of A and B; products are exact and accumulation is f32 (MFMA).  dtype_out is the storage
 *   type of C (SP_F32, or the same 16-bit type as the input).  bias (N,) f32 may be NULL.
 *   alpha must be non-zero (kernel.spi:49).  beta == 0 means C is never read, so NaNs in the
 *   old C do not propagate (kernel.spi:152-154).
 *   K must be a multiple of 8 (16-bit) / 4 (f32): rows of A and B are whole 16-byte chunks.  Every such
 *   shape with N a multiple of 4 runs on the tiled MFMA kernels (tiles that overhang M, N or K are
 *   masked); only N not a multiple of 4 falls back to a slow one-thread-per-output kernel.
 */
int sp_gemm_abt(int dtype_in, int dtype_out, const void* A, const void* B, void* C, const float* bias,
                int64_t M, int64_t N, int64_t K, float alpha, float beta, uint32_t flags, void* stream);

/*
 * `batch` independent products C_e = alpha * A_e . B_e^T + beta * C_e [+ bias] [ReLU] in one launch:
 * member e starts stride_a / stride_b / stride_c ELEMENTS after member e - 1 (0 = every member
 * uses the same A or B).  Replaces the loop over `.ensemble` that `graph_run_host model {ensemble}`
 * makes around `BlockMatmul(x, apply .ensemble weights)` for `matmul_ensemble` layers
 * (ml/layers.spi:227-240,336-344,468-471): A = the shared input, stride_a = 0, B = the (E, out, in)
 * weight tensor, stride_b = out * in.  The tile is chosen for the whole batch, so many small members
 * fill the chip.  bias (N,) is shared by all members.
 */
int sp_gemm_abt_batched(int dtype_in, int dtype_out, const void* A, const void* B, void* C, const float* bias,
                        int64_t M, int64_t N, int64_t K, int64_t batch, int64_t stride_a, int64_t stride_b,
                        int64_t stride_c, float alpha, float beta, uint32_t flags, void* stream);

/* Which tile configuration sp_gemm_abt picks for a shape (the counterpart of
 * `matmul_config_tf32`, ml/matmul/run.spi:8-19).  Writes block tile sizes and the workgroup size;
 * tile_m == 0 means the general kernel. */
int sp_gemm_config(int dtype_in, int64_t M, int64_t N, int64_t K,
                   int32_t* tile_m, int32_t* tile_n, int32_t* tile_k, int32_t* threads);

/* ------------------------------------------------------------------------------------------ */
/* Row primitives                                                                              */
/* ------------------------------------------------------------------------------------------ */

/*
 * Fused row pipeline over logits (rows, cols) f32: row max, sum of exp(x - max), softmax,
 * inclusive prefix sum of the probabilities, argmax, and inverse-CDF sampling with one uniform
 * u[row] in (0, 1] per row.  One pass over HBM; any output pointer may be NULL to skip it.
 *
 * Replaces the chain row_reduce(local_argmax) / row_map(local_softmax + local_inclusive_scan_sum) /
 * row_map_reduce(local_softmax_and_discrete_sampling) of ml/primitives.spi:514-536,705-716,782-802
 * (test2, :925-955).  Sampling rule (:782-798): m = max cdf over p > 0; result = smallest j with
 * p_j > 0 and cdf_j >= u * m.  argmax ties resolve to the lowest index.
 * cols: multiple of 4, 4 <= cols <= 1024.  flags is reserved and must be 0.
 */
int sp_row_ops(const float* logits, const float* u, float* rowmax, float* rowsum, float* probs, float* cdf,
               int32_t* argmax, int32_t* sample, int64_t rows, int64_t cols, uint32_t flags, void* stream);

typedef enum {
    SP_ROW_IDENTITY = 0,                /* row_map (fun config x i j_tns => x)          primitives.spi:930 */
    SP_ROW_SOFTMAX = 1,                 /* local_softmax                                primitives.spi:711-716 */
    SP_ROW_MASKED_SOFTMAX = 2,          /* local_masked_softmax, mask j < mask_size     primitives.spi:748-759 */
    SP_ROW_LN_L2 = 3,                   /* local_ln_l2                                  primitives.spi:701-703 */
    SP_ROW_REGRET_MATCHING = 4,         /* local_regret_matching                        primitives.spi:718-722 */
    SP_ROW_MASKED_REGRET_MATCHING = 5,  /* local_masked_regret_matching                 primitives.spi:761-780 */
    SP_ROW_INCLUSIVE_SCAN = 6,          /* local_inclusive_scan_sum                     primitives.spi:323-325 */
    SP_ROW_EXCLUSIVE_SCAN = 7,          /* local_exclusive_scan config 0 (+)            primitives.spi:327 */
    SP_ROW_L1_NORMALIZE = 8             /* local_l1_normalize (sp_row_l1_normalize only) primitives.spi:725-729 */
} sp_row_op;

/* out = op(x) row by row, x and out (rows, cols) f32.  Replaces `row_map f x out`
 * (ml/primitives.spi:514-520) for the lambdas listed in sp_row_op.  mask_size is used by the
 * masked ops only (1 <= mask_size <= cols). */
int sp_row_map_f32(int op, const float* x, float* out, int64_t rows, int64_t cols, int32_t mask_size, void* stream);

/* out = |x| * (s > threshold ? threshold / s : 1) row by row, s = sum over j of |x[r, j]|: a row whose l1 norm is above
 * `threshold` (> 0) is scaled down to it, any other row becomes its absolute values.  Replaces
 * `row_map (local_l1_normalize threshold)` (ml/primitives.spi:725-729; caller ml/cfr.spi:244, the decay of the average
 * policy).  `out` may be x. */
int sp_row_l1_normalize(const float* x, float* out, int64_t rows, int64_t cols, float threshold, void* stream);

/* Integer scans (SP_ROW_INCLUSIVE_SCAN / SP_ROW_EXCLUSIVE_SCAN / SP_ROW_IDENTITY) on i32 rows; exact
 * (wrap-around two's complement like the device adds of the reference, test2 :948-950). */
int sp_row_map_i32(int op, const int32_t* x, int32_t* out, int64_t rows, int64_t cols, void* stream);

/* How a sampling op obtains its uniforms when no `u` tensor is given: the reference's device-side
 * Philox4_32_10 stream (corecuda/random.spi:22-32,84) with curand_init(seed, subsequence, 0). */
typedef enum {
    SP_PHILOX_BLOCK = 0,   /* row_map_reduce: subsequence = thread-in-block        primitives.spi:927 */
    SP_PHILOX_GRID = 1,    /* grid_row_map_reduce: subsequence = thread-in-grid    primitives.spi:1014,493 */
    SP_PHILOX_GATHER = 2,  /* row_gather_reduce: one row per thread                primitives.spi:409-413 */
    SP_PHILOX_LAYER = 3    /* graph_run_host: the tensor is (blocks, rows_per_block, cols), block b works
                              through its own slice, subsequence = thread-in-grid       layers.spi:339-344 */
} sp_philox_mode;

typedef struct {
    uint64_t seed;               /* reference: 12344321 (corecuda/cupy.spi:6) */
    uint64_t offset;             /* 32-bit draws every thread has already consumed: the reference keeps one
                                    generator state per thread for a whole graph run, and every sampling
                                    node advances it by 4 draws per row-iteration (layers.spi:341) */
    int32_t mode;                /* sp_philox_mode */
    int32_t threads_per_block;   /* reference: 256 */
    int32_t blocks_per_grid;     /* reference: 24 (RTX 4060) or 112 (H100), corecuda/base.spi:14-42 */
    int32_t rows_per_block;      /* SP_PHILOX_LAYER only: rows of one block's slice */
    int64_t member_rows;         /* 0, or: the rows are `rows / member_rows` stacked runs of the same op (the
                                    members of an ensemble evaluated in one launch); row r then draws what row
                                    r % member_rows of a run starting at offset + (r / member_rows) * member_draws
                                    would draw */
    uint64_t member_draws;       /* draws every thread consumes per run: all sampling nodes of the graph */
} sp_philox_t;

/*
 * probs = op(x) (op in IDENTITY, SOFTMAX, MASKED_SOFTMAX, REGRET_MATCHING, MASKED_REGRET_MATCHING),
 * then sample = local_discrete_sampling(probs).  Replaces `row_map_reduce
 * (local_softmax_and_discrete_sampling rng) x probs sample` and its masked / regret-matching
 * siblings (ml/primitives.spi:528-536,800-814).  Exactly one of `u` (rows,) f32 in (0,1] and
 * `philox` must be given.  probs_out, cdf_out, u_out (the uniform each row used) and prob_out may be
 * NULL.  prob_out (rows,) receives the probability of the sampled index, which is what
 * `local_get_prob config action_id (zip probs j_tns)` returns next to the action in the agents'
 * `get_action` (ml/cem.spi:152-164, ml/cfr.spi:117-129); 0 for a row without positive mass.
 */
int sp_row_sample(int op, const float* x, const float* u, const sp_philox_t* philox, float* probs_out, float* cdf_out,
                  float* u_out, int32_t* sample_out, float* prob_out, int64_t rows, int64_t cols, int32_t mask_size,
                  void* stream);

/*
 * u_out[r] = the uniform in (0, 1] that row r of a (rows, cols) sampling op draws from the stream
 * `philox` describes: the reference's `random.init` + `random.uniform` (corecuda/random.spi:22-32,84)
 * without the op around it, for callers that feed the uniforms to sp_mlp_forward or sp_row_ops.
 */
int sp_philox_uniforms(const sp_philox_t* philox, float* u_out, int64_t rows, int64_t cols, void* stream);

/*
 * prob_out[r] = op(x)[r, action[r]]: `row_gather_reduce` of `local_get_prob` after an optional
 * (masked) softmax / regret matching (ml/primitives.spi:824-830; callers ml/cfr.spi:97-107).  The
 * reference asserts that the action id is a column of the row; here an id outside [0, cols) gives 0.
 */
int sp_row_get_prob(int op, const float* x, const int32_t* action, float* prob_out, int64_t rows, int64_t cols,
                    int32_t mask_size, void* stream);

/*
 * out[r] = (OR over j of (not (x[r, j] <= 0)) << j) mod modulo: `local_binarize` (ml/primitives.spi:817-821),
 * the hash head `binarize` of ml/layers.spi:439-446; like there a NaN sets its bit.  The shift is the
 * device's 32-bit shift: columns j >= 32 contribute nothing.  modulo must be positive.
 */
int sp_row_binarize(const float* x, uint32_t* out, int64_t rows, int64_t cols, uint32_t modulo, void* stream);

/*
 * Cross-entropy-method update of one layer's weights (ml/cem.spi:99-117, `cem`): weights_t is the
 * TRANSPOSED weight tensor (rows = weight positions, ensemble columns, what `grid_transpose`
 * produces, :131-132); winners (mask[e] != 0) keep their value, every other member is redrawn as
 * (normals[r, e] * max(std, noise) + mean) * decay with mean / std taken over the winners of the
 * row (std = biased std * n / (n - 1), 0 for a single winner).  The reference draws `normals`
 * from curand_normal on the fly; here the caller supplies standard normals (rows, ensemble), or calls
 * sp_cem_resample_philox below.
 * `out` may be weights_t.  The reference uses noise 0.1, decay 1 (:76-78).
 */
int sp_cem_resample(const float* weights_t, const int32_t* mask, const float* normals, float* out, int64_t rows,
                    int64_t ensemble, float noise, float decay, void* stream);

/*
 * sp_cem_resample with the normals drawn on the device, as the reference does (`random.normal rng`, ml/cem.spi:113,
 * corecuda/random.spi:85: curand_normal on a Philox4_32_10 state): row r takes the sequence curand_normal yields for
 * curand_init(seed, subsequence = r, offset), i.e. columns 4 g .. 4 g + 3 are the two Box-Muller pairs of 4-draw
 * group offset / 4 + g.  `offset` (a multiple of 4) lets successive updates continue the stream.  Which thread
 * draws for which weight is a property of the reference's launch geometry and its fast sincos, neither of which this
 * build shares: the mapping above is this build's own and the values are not bit-comparable with the reference's.
 */
int sp_cem_resample_philox(const float* weights_t, const int32_t* mask, uint64_t seed, uint64_t offset, float* out,
                           int64_t rows, int64_t ensemble, float noise, float decay, void* stream);

/*
 * `grid_update_rewards_mask` (ml/cem.spi:92-96): rewards is (ensemble, 2) f32 pairs (reward sum,
 * count); mask[e] = (count ? reward / count : 0) >= average over the ensemble; the pairs are zeroed.
 */
int sp_cem_update_mask(float* rewards, int32_t* mask, int64_t ensemble, void* stream);

typedef enum { SP_REDUCE_SUM = 0, SP_REDUCE_PROD = 1, SP_REDUCE_MAX = 2, SP_REDUCE_MIN = 3, SP_REDUCE_AVERAGE = 4 } sp_reduce_op;
typedef enum { SP_MAP_IN_IDENTITY = 0, SP_MAP_IN_SQUARE = 1, SP_MAP_IN_ABS = 2 } sp_map_in;
typedef enum { SP_MAP_OUT_IDENTITY = 0, SP_MAP_OUT_SQRT = 1 } sp_map_out;

/*
 * out[r] = map_out(reduce over j of map_in(x[r, j])), x (rows, cols) f32, out (rows,) f32; cols any multiple of 4.
 * Replaces `row_reduce` of `local_sum` / `local_prod` / `local_max` / `local_min` / `local_average`
 * (ml/primitives.spi:330-348,523-526), `reduce_2d` and `map_reduce_map_2d map_in neutral f map_out from to`
 * (ml/primitives.spi:593-660) for the lambdas in the enums above; `grid_map_reduce_map_2d grid sqr 0 (+) sqrt` is the
 * per-row weight norm of the CEM update (ml/cem.spi:139).  The neutral elements are the reference's (0, 1, -inf, +inf);
 * `local_length` is cols.  The order of a float sum depends on cols only.
 */
int sp_row_reduce_f32(int op, int map_in, int map_out, const float* x, float* out, int64_t rows, int64_t cols, void* stream);

typedef enum { SP_MAP_COPY = 0, SP_MAP_RELU = 1, SP_MAP_TANH = 2, SP_MAP_SIGMOID = 3 } sp_map_op;

/* out[i] = f(x[i]) over n f32 elements (n multiple of 4).  Replaces `primitives.map f from to`
 * (ml/primitives.spi:115-133) for the activation lambdas of ml/layers.spi:353-355. */
int sp_map_f32(int op, const float* x, float* out, int64_t n, void* stream);

/* out[0] = x[0] op x[1] op ... op x[n - 1] over a whole tensor, one launch over the whole device.  op: SP_REDUCE_SUM,
 * SP_REDUCE_PROD, SP_REDUCE_MAX or SP_REDUCE_MIN with the neutral elements 0, 1, lowest and highest value of the type
 * (corebase/limit.spi); dtype: 0 = f32, 1 = i32, 2 = u64.  float max / min ignore a NaN operand unless both are NaN.
 * Replaces `reduce neutral f` / `grid_reduce grid neutral f` (ml/primitives.spi:136-197; `grid_reduce grid 0 max`,
 * ml/cem.spi:140; `reduce 0 (+)` on u64, test6 :1102-1105).
 * `workspace` must hold at least sp_reduce_workspace_bytes() bytes of device memory (per-block partial results, each
 * tagged with a number drawn per launch, and a give-up counter; no allocation here).  Zero-fill it once before its
 * first use (the counter starts from what it finds; the slots do not depend on it: a partial result only counts when
 * it carries the tag of the launch that polls it).  Calls that may run at the same time need a workspace each.  The
 * order of the operations depends on n only, so an f32 result is the same from run to run.
 * The launch ends with one workgroup waiting for the others' partial results.  That wait is bounded (5 ms unless
 * sp_reduce_set_poll_limit changed it): when other work keeps part of the launch off the device for longer, the call
 * gives up, out[0] becomes a NaN (f32) or an all-ones word, the slots are cleared and the workspace's give-up counter
 * goes up by one.  sp_reduce_status reads that counter (it copies 8 bytes to the host and therefore WAITS for the
 * stream, the only call of this library that does); a caller that cannot rule out such contention checks it.
 * sp_reduce_set_poll_limit sets the bound in microseconds for later launches of this process (0 = the default, at most
 * 10 s; a negative value makes every launch give up without waiting: a way to exercise the give-up path in which
 * every kernel still runs to its end). */
int sp_reduce(int op, int dtype, const void* x, void* out, int64_t n, void* workspace, int64_t workspace_bytes, void* stream);
/* sp_reduce with op = SP_REDUCE_SUM. */
int sp_reduce_sum(int dtype, const void* x, void* out, int64_t n, void* workspace, int64_t workspace_bytes, void* stream);
int64_t sp_reduce_workspace_bytes(void);
int sp_reduce_status(const void* workspace, int64_t workspace_bytes, int64_t* give_ups, void* stream);
int sp_reduce_set_poll_limit(int64_t microseconds);

/* sp_reduce_sum for callers that cannot allocate device memory or hand over a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The
 * partial sums and their valid marks live in a 16 KiB + 16 B array (the marked slots and the give-up counter) inside
 * the library's own device image, one copy per GPU, kept until the process ends; the call allocates nothing and uses no memset.  Same kernel, same grid and
 * therefore bit-identical results to sp_reduce_sum.  n must not exceed sp_reduce_sum_static_max_n() (2^36
 * elements), else SP_ERR_SHAPE.  All calls on one GPU share the array: calls that may overlap in time (different
 * streams, different threads) race and must be serialised by the caller. */
int sp_reduce_sum_static(int dtype, const void* x, void* out, int64_t n, void* stream);
int64_t sp_reduce_sum_static_max_n(void);

/* to[a][c][b] = from[a][b][c] for 4-byte elements.  Replaces `grid_transpose_snd`
 * (ml/primitives.spi:36-112, test5 :1078-1088). */
int sp_transpose_inner_b32(const void* from, void* to, int64_t a, int64_t b, int64_t c, void* stream);

/* ------------------------------------------------------------------------------------------ */
/* Dense layers                                                                                */
/* ------------------------------------------------------------------------------------------ */

typedef enum {
    SP_HEAD_NONE = 0,            /* policy_out receives the last layer's outputs */
    SP_HEAD_SOFTMAX = 1,         /* softmax                          ml/layers.spi:370-375 */
    SP_HEAD_REGRET_MATCHING = 2, /* regret_matching                  ml/layers.spi:377-382 */
    SP_HEAD_SOFTMAX_RM = 3       /* softmax, then regret matching of the probabilities */
} sp_head;

/*
 * Fused forward pass of a dense stack: h_0 = x; h_{i+1} = relu(h_i . W_i^T [+ b_i]) for all but the
 * last layer; policy = head(h_{n-1} . W_{n-1}^T [+ b_{n-1}]); action = discrete sample of policy
 * with u[row].  One kernel; activations never leave the CU.
 *
 * Replaces the interpreter chain block_matmul -> block_map(relu) -> ... -> block_row_map_reduce
 * (ml/layers.spi:194-240; generated ml/layers.py:4531-4546, launched through
 * `entry0(weights, workspace, adjoint)`, ml/layers.py:4500,5894), where every arrow is a round
 * trip through the global-memory workspace.
 *
 *   dtype        SP_F16 or SP_BF16: storage type of x and of every weight matrix
 *   x            (batch, dims[0])
 *   weights[i]   (dims[i+1], dims[i]) row-major = the B operand of A.B^T (ml/layers.spi:467);
 *                `weights` is a HOST array of n_layers device pointers
 *   biases       NULL, or a host array of n_layers device pointers to f32 (dims[i+1],) (entries may be NULL)
 *   dims         host array of n_layers + 1 layer widths; dims[0] a multiple of 16, hidden widths
 *                multiples of 32, all <= 256; dims[n_layers] <= 64
 *   u            (batch,) f32 in (0, 1], or NULL
 *   philox       NULL, or the stream the head draws its uniforms from itself, as the reference's graph run does
 *                (one generator per thread seeded at the start of the run, ml/layers.spi:339-344; the struct and its
 *                row -> draw mappings are those of sp_row_sample, SP_PHILOX_LAYER being the graph run's): row r uses
 *                exactly the uniform sp_philox_uniforms(philox, ., batch, dims[n_layers]) would hand out for it, so no
 *                uniform tensor is written or read.  dims[n_layers] must then be a multiple of 4 (the row width of
 *                the reference's sampling op).  With action_out exactly one of u and philox is given.
 *   policy_out   (batch, dims[n_layers]) f32
 *   action_out   (batch,) i32 or NULL
 *   logits_out   (batch, dims[n_layers]) f32 or NULL
 *   mask_size    0 = no mask, else the head only considers columns j < mask_size (ml/layers.spi:408-432)
 *
 * Accuracy: hidden activations are rounded to `dtype` between layers (they are the next MFMA's operands).
 * Against an f32 evaluation of the same rounded inputs and weights that keeps its activations in f32, the
 * policy stays within a relative Frobenius error of 3e-3 for both types and so do f16 logits; the raw
 * logits_out of a BF16 stack (8 significant bits per hidden activation and layer) are only held to 1e-2.
 * Against an evaluation that rounds its activations the same way everything is within 2e-4.
 */
int sp_mlp_forward(int dtype, const void* x, int32_t n_layers, const void* const* weights, const float* const* biases,
                   const int32_t* dims, const float* u, const sp_philox_t* philox, float* policy_out, int32_t* action_out,
                   float* logits_out, int64_t batch, int32_t head, int32_t mask_size, void* stream);

/*
 * The same forward pass over weights that were packed once into MFMA operand order: the weights then stream
 * from global memory straight into registers, every load of a launch in flight from its first cycle, instead of
 * through an LDS ring (config 3: 8.5 us -> see the bench).  Build extension; the reference keeps its weights
 * row-major in the weights arena (ml/layers.spi:127-179) and has no counterpart.
 *
 *   sp_mlp_packed_bytes   size of the packed buffer for a stack, 0 when the packed kernel does not take it:
 *                         3 to 5 layers, every hidden width 256, dims[0] a multiple of 16 and <= 256,
 *                         dims[n_layers] <= 64
 *   sp_mlp_pack_weights   writes `packed` (caller memory, 16-byte aligned, at least sp_mlp_packed_bytes) from
 *                         the row-major `weights` of sp_mlp_forward; one small launch, nothing is allocated.
 *                         Has to be repeated whenever the weights change; the packed buffer holds no pointers.
 *                         Of an output layer wider than 16 only the first 16 rows are packed.
 *   sp_mlp_forward_packed sp_mlp_forward with `packed` in place of `weights`; same results (the k-order of the
 *                         sums is the same).  At most 16 outputs: dims[n_layers] <= 16, or a masked head of at
 *                         most 16 columns without logits_out.  SP_ERR_UNSUPPORTED for any other stack: call
 *                         sp_mlp_forward with the row-major weights instead.  `packed_bytes` is the size the buffer
 *                         was packed with and must equal sp_mlp_packed_bytes(n_layers, dims), else SP_ERR_ARG: a
 *                         buffer packed for another layer count or another class of first width has another size
 *                         and would be read out of bounds.  The buffer does not record the 16-bit type or the
 *                         weights' values: handing over a buffer packed from other weights of the same shape is
 *                         the caller's to avoid.
 */
int64_t sp_mlp_packed_bytes(int32_t n_layers, const int32_t* dims);
int sp_mlp_pack_weights(int dtype, int32_t n_layers, const void* const* weights, const int32_t* dims, void* packed,
                        int64_t packed_bytes, void* stream);
int sp_mlp_forward_packed(int dtype, const void* x, int32_t n_layers, const void* packed, int64_t packed_bytes,
                          const float* const* biases, const int32_t* dims, const float* u, const sp_philox_t* philox,
                          float* policy_out, int32_t* action_out, float* logits_out, int64_t batch, int32_t head,
                          int32_t mask_size, void* stream);

/* Fused forward of an ENSEMBLE of one- or two-layer f32 stacks on one shared input, one launch:
 *   n_layers = 2:  policy[e] = head(relu(x . W1[e]^T) . W2[e]^T)
 *   n_layers = 1:  policy[e] = head(x . W1[e]^T),                 e = 0 .. members - 1
 * x: (batch, dims[0]) f32; weights[i]: (members, dims[i + 1], dims[i]) f32, the stacked tensors of `matmul_ensemble`
 * (ml/layers.spi:468-479).  Two layers: dims[0] a multiple of 8 in [8, 128], dims[1] = 64; one layer: dims[0] a
 * multiple of 8 in [8, 256].  Output width dims[n_layers] <= 64; dtype = SP_F32.  head / mask_size as for
 * sp_mlp_forward, with at most 4 computed outputs (the output width, or mask_size of a masked head; the columns behind
 * the mask are written as zeros).
 * policy_out: (members, batch, dims[n_layers]); action_out: (members, batch) or NULL; u: (members, batch) uniforms in
 * (0, 1] or NULL; philox: a stream over the members x batch stacked rows (member_rows = batch) or NULL; at most one
 * of u and philox, one of them when action_out is given.
 * Replaces: `graph_run_host model {ensemble}` (ml/layers.spi:336-344, the interpreter of :194-240 run member by
 * member) for the graphs of the reference's CEM policies: game/leduc/model_cem.spi:55-63
 * (input -> matmul_ensemble_with_adjoint -> relu -> matmul_ensemble_with_adjoint -> masked_regret_matching') and
 * game/nl_hu_holdem/model_cem.spi:84-100 (input -> matmul_ensemble_with_adjoint -> masked_regret_matching'). */
int sp_mlp_forward_ensemble(int dtype, const void* x, int32_t n_layers, const void* const* weights, const int32_t* dims,
                            int32_t members, const float* u, const sp_philox_t* philox, float* policy_out,
                            int32_t* action_out, int64_t batch, int32_t head, int32_t mask_size, void* stream);

/* out[e][r] = (OR over j of (not (y[r, j] <= 0)) << j) mod modulo with y = x . W[e]^T: one ensemble layer and the hash
 * head `binarize` in one launch; y is never written.  x: (batch, k0) f32, k0 a multiple of 8 in [8, 256]; weights:
 * (members, n, k0) f32; out: (members, batch) u32.  As in sp_row_binarize the shift is the device's 32-bit shift
 * (columns j >= 32 contribute nothing, so only the first 32 rows of every W[e] are read) and a NaN sets its bit.
 * Replaces: `graph_run_host model {ensemble}` for input -> matmul_ensemble -> binarize' (the reference's CFR
 * models, game/leduc/model_cfr.spi:56-61, game/nl_hu_holdem/model_cfr.spi:82-88; ml/layers.spi:439-446,
 * ml/primitives.spi:817-821). */
int sp_ensemble_binarize(int dtype, const void* x, const void* weights, uint32_t* out, int32_t members, int64_t batch,
                         int32_t k0, int32_t n, uint32_t modulo, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SPIRAL_MI355_H */
