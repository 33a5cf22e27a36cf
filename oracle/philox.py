"""Philox4x32-10 and curand_uniform restated on the CPU.  TEST INFRASTRUCTURE ONLY.

The reference draws its uniforms on the device from `curandStatePhilox4_32_10_t`
(corecuda/random.spi:9,22-32) with `curand_init(seed, subsequence, offset)` and
`curand_uniform` (corecuda/random.spi:84); seed = 12344321 (corecuda/cupy.spi:6).  cuRAND is
a third-party dependency that is not part of the reference tree; this file restates the
published Philox-4x32-10 algorithm (Salmon et al., "Parallel random numbers: as easy as
1, 2, 3", SC'11) and cuRAND's documented counter layout:

    key     = (seed_lo, seed_hi)
    counter = (n_lo, n_hi, subsequence_lo, subsequence_hi)    n = index of the 4-word group
    curand() hands out words x, y, z, w of group n in that order, then moves to group n+1
    curand_uniform(x) = x * 2^-32 + 2^-33   (computed in f32, result in (0, 1])

Pinned by the Random123 known-answer vectors and by replaying every sampled index held in
the reference's golden outputs (tests/test_oracle_golden.py).
"""
import numpy as np

PHILOX_M0 = np.uint64(0xD2511F53)
PHILOX_M1 = np.uint64(0xCD9E8D57)
PHILOX_W0 = 0x9E3779B9
PHILOX_W1 = 0xBB67AE85
CONSTANT_SEED = 12344321  # corecuda/cupy.spi:6

_MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(ctr, key):
    """ctr: (..., 4) uint32, key: (..., 2) uint32 -> (..., 4) uint32 after 10 rounds."""
    ctr = np.asarray(ctr, dtype=np.uint64)
    key = np.asarray(key, dtype=np.uint64)
    c0, c1, c2, c3 = (ctr[..., i].copy() for i in range(4))
    k0, k1 = key[..., 0].copy(), key[..., 1].copy()
    for r in range(10):
        if r:
            k0 = (k0 + np.uint64(PHILOX_W0)) & _MASK32
            k1 = (k1 + np.uint64(PHILOX_W1)) & _MASK32
        p0 = PHILOX_M0 * c0
        p1 = PHILOX_M1 * c2
        hi0, lo0 = p0 >> np.uint64(32), p0 & _MASK32
        hi1, lo1 = p1 >> np.uint64(32), p1 & _MASK32
        c0, c1, c2, c3 = hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0
    return np.stack([c0, c1, c2, c3], axis=-1).astype(np.uint32)


def curand_words(seed, subsequence, draw_index):
    """The `draw_index`-th (0-based) 32-bit output of curand() for a Philox state initialised
    with curand_init(seed, subsequence, offset=0).  `subsequence` and `draw_index` broadcast."""
    subsequence = np.asarray(subsequence, dtype=np.uint64)
    draw_index = np.asarray(draw_index, dtype=np.uint64)
    subsequence, draw_index = np.broadcast_arrays(subsequence, draw_index)
    group = draw_index >> np.uint64(2)
    ctr = np.stack([group & _MASK32, group >> np.uint64(32),
                    subsequence & _MASK32, subsequence >> np.uint64(32)], axis=-1)
    key = np.empty(ctr.shape[:-1] + (2,), dtype=np.uint64)
    key[..., 0] = np.uint64(seed & 0xFFFFFFFF)
    key[..., 1] = np.uint64((seed >> 32) & 0xFFFFFFFF)
    out = philox4x32_10(ctr, key)
    word = (draw_index & np.uint64(3)).astype(np.int64)
    return np.take_along_axis(out, word[..., None], axis=-1)[..., 0]


def curand_uniform(words):
    """uint32 -> f32 in (0, 1], cuRAND's mapping, evaluated in f32 like the device does."""
    w = np.asarray(words, dtype=np.uint32).astype(np.float32)  # RNE u32 -> f32, as the device cvt
    return w * np.float32(2.3283064e-10) + np.float32(1.1641532e-10)


def row_uniforms_block(rows, cols, seed=CONSTANT_SEED, threads_per_block=256):
    """Uniform used by each row of a block-level `row_map_reduce` sampling op
    (ml/primitives.spi:786-791 with rng subsequence = thread-in-block, :927).  Every thread
    draws one uniform per element it holds (4 for f32) and the reduction keeps the draw that is
    attached to column 0, i.e. the first draw of the row's lane 0 in that row-iteration."""
    t = cols // 4
    r_per_iter = threads_per_block // t
    r = np.arange(rows)
    return curand_uniform(curand_words(seed, (r % r_per_iter) * t, 4 * (r // r_per_iter)))


def row_uniforms_grid(rows, cols, seed=CONSTANT_SEED, threads_per_block=256, blocks=24):
    """Same for `grid_row_map_reduce` (subsequence = thread-in-grid, ml/primitives.spi:1014;
    row-iterations are block-strided, :493)."""
    t = cols // 4
    r_per_iter = threads_per_block // t
    r = np.arange(rows)
    it = r // r_per_iter
    sub = (it % blocks) * threads_per_block + (r % r_per_iter) * t
    return curand_uniform(curand_words(seed, sub, 4 * (it // blocks)))


def row_uniforms_gather(n_threads, cols, seed=CONSTANT_SEED, threads_per_block=256):
    """Same for `row_gather_reduce`, where every *thread* owns one short row and the block
    transposes them through shared memory (corecuda/transposing_loop.spi:80-91)."""
    t_per_row = cols // 4
    d = threads_per_block // t_per_row
    t = np.arange(n_threads)
    lt = t % threads_per_block
    sub = (t // threads_per_block) * threads_per_block + (lt % d) * t_per_row
    return curand_uniform(curand_words(seed, sub, 4 * (lt // d)))


def row_uniforms_layer(blocks, rows_per_block, cols, seed=CONSTANT_SEED, threads_per_block=256, offset=0):
    """Same for a sampling node of a layer graph run by `graph_run_host` (ml/layers.spi:339-344):
    the tensor is (blocks, rows_per_block, cols), block b works through its own slice with the
    block-level `row_map_reduce`, the generator is seeded once per thread with subsequence =
    thread-in-grid and keeps its state for the whole run, so a node starts `offset` draws in
    (4 per row-iteration of every earlier sampling node).  Returns (blocks * rows_per_block,)."""
    t = cols // 4
    r_per_iter = threads_per_block // t
    b = np.repeat(np.arange(blocks), rows_per_block)
    r = np.tile(np.arange(rows_per_block), blocks)
    sub = b * threads_per_block + (r % r_per_iter) * t
    return curand_uniform(curand_words(seed, sub, offset + 4 * (r // r_per_iter)))


def draws_per_sampling_node(rows_per_block, cols, threads_per_block=256):
    """32-bit draws one sampling node takes from every thread's generator: 4 per row-iteration."""
    r_per_iter = threads_per_block // (cols // 4)
    return 4 * ((rows_per_block + r_per_iter - 1) // r_per_iter)


def curand_normal_rows(rows, cols, seed=CONSTANT_SEED, offset=0):
    """Standard normals as `curand_normal` (corecuda/random.spi:85) hands them out: row r is the sequence of
    a Philox state initialised with curand_init(seed, subsequence = r, offset); successive draws come in
    Box-Muller pairs from two 32-bit words x, y:
        u = x * 2^-32 + 2^-33,  v = y * (2^-32 * 2 pi) + 2^-33 * 2 pi,  (sqrt(-2 ln u) sin v, sqrt(-2 ln u) cos v)
    (cuRAND's `_curand_box_muller`, restated from its published header; evaluated in f32).  This is the stream
    sp_cem_resample_philox draws from.  PARITY UNPINNED against the reference: it assigns draws to weights by its
    launch geometry and evaluates sin/cos/log with the fast intrinsics of its platform; no output of it exists."""
    assert cols % 2 == 0 and offset % 4 == 0
    r = np.repeat(np.arange(rows), cols)
    j = np.tile(np.arange(cols), rows)
    x = curand_words(seed, r, offset + (j // 2) * 2).astype(np.float32)
    y = curand_words(seed, r, offset + (j // 2) * 2 + 1).astype(np.float32)
    two_pi = np.float32(2.3283064e-10) * np.float32(6.2831855)
    u = x * np.float32(2.3283064e-10) + np.float32(1.1641532e-10)
    v = y * two_pi + two_pi * np.float32(0.5)
    s = np.sqrt(np.float32(-2.0) * np.log(u)).astype(np.float32)
    out = np.where(j % 2 == 0, s * np.sin(v).astype(np.float32), s * np.cos(v).astype(np.float32))
    return out.astype(np.float32).reshape(rows, cols)
