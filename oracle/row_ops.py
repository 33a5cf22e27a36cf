"""Row primitives restated in NumPy (f32 / i32 arithmetic).  TEST INFRASTRUCTURE ONLY.

Follows ml/primitives.spi: every function below acts on the innermost dimension of a
row-major (rows, cols) tensor, exactly like the user lambdas that `row_map`, `row_reduce`
and `row_map_reduce` (ml/primitives.spi:423-590) run on one row at a time.

Float summation order.  The reference sums a row as: sequentially over the 4 elements a
thread holds, then a butterfly / scan across the threads of the row
(ml/primitives.spi:295-348, corecuda/cooperative_groups.spi:58-80); the order inside the
cooperative-groups collectives is not specified by CUDA.  Two orders are offered here:

  order="sequential"  left-to-right f32 accumulation (np.cumsum), the textbook reading
  order="wave"        the association the HIP kernels use, restated exactly so that the
                      cumulative distribution (and therefore the sampled index) can be
                      compared bit for bit:
                        lane t owns columns 4t..4t+3 of each 4*T-column chunk (T lanes per row)
                        s_t   = ((x0 + x1) + x2) + x3
                        incl  = inclusive scan of s over the T lanes:
                                Hillis-Steele inside rows of min(T, 16) lanes
                                  (for d = 1, 2, 4, 8: v_t += v_{t-d} for t >= d, t in the row);
                                T >= 32: each lane of an odd 16-lane row adds the last value of
                                  the row before it;
                                T == 64: each lane of rows 2 and 3 then adds the value lane 31
                                  holds after the previous step
                        start = carry + (incl_{t-1} or 0);  out_k = (...(start + x0) + ...) + x_k
                        carry = carry + incl_{T-1}                      (next chunk)
"""
import numpy as np

INT_MAX = np.int32(2147483647)  # corebase/limit.spi, neutral element of `min` on i32
F32 = np.float32


def _f32(x):
    return np.ascontiguousarray(x, dtype=np.float32)


def lanes_per_row(cols):
    """Lanes that share one row in the kernels.  Up to 64 columns: one lane per 4 columns, rounded
    up to a power of two.  Up to 256 columns: 16 lanes, each with one 4-column piece of every
    64-column chunk.  Wider rows: 64 lanes, one piece per 256-column chunk."""
    if cols > 256:
        return 64
    t = 1
    while t * 4 < cols and t < 16:
        t *= 2
    return t


# ----------------------------------------------------------------------------------------------
# reductions
# ----------------------------------------------------------------------------------------------

def reduce_sum(x):
    """`reduce 0 (+)` over a whole tensor (ml/primitives.spi:136-197).  Exact for integers."""
    x = np.asarray(x)
    if x.dtype.kind in "iu":
        return x.sum(dtype=x.dtype)
    return np.float32(x.astype(np.float64).sum())


def row_max(x):
    """`local_max` (ml/primitives.spi:346)."""
    return _f32(x).max(axis=-1)


def row_sum(x):
    """`local_sum` (ml/primitives.spi:338); f64 accumulation rounded once, compare to tolerance."""
    return _f32(x).sum(axis=-1, dtype=np.float64).astype(np.float32)


def row_reduce(x, op="sum", map_in="identity", map_out="identity"):
    """`row_reduce` of `local_sum` / `local_prod` / `local_max` / `local_min` / `local_average`
    (ml/primitives.spi:330-348) and `map_reduce_map_2d map_in neutral f map_out` (:593-660) along the innermost
    dimension.  Sums and products accumulate in f64 and are rounded once: compare to a tolerance."""
    x = _f32(x).astype(np.float64)
    x = {"identity": x, "square": x * x, "abs": np.abs(x)}[map_in]
    r = {"sum": x.sum(axis=-1), "prod": x.prod(axis=-1), "max": x.max(axis=-1), "min": x.min(axis=-1),
         "average": x.sum(axis=-1) / x.shape[-1]}[op]
    if map_out == "sqrt":
        r = np.sqrt(r)
    return r.astype(np.float32)


def argmax(x):
    """`local_argmax` (ml/primitives.spi:705-708).  The reference keeps `a` when `a.v > b.v` in a
    butterfly whose operand order is unspecified, so ties are arbitrary there; this build fixes
    the lowest index, which is np.argmax."""
    return np.argmax(_f32(x), axis=-1).astype(np.int32)


# ----------------------------------------------------------------------------------------------
# row maps
# ----------------------------------------------------------------------------------------------

def softmax(x, shift="max"):
    """`local_softmax` (ml/primitives.spi:711-716).  The reference shifts by the row *mean*
    (author's TODO at :712); shifting by the max is the same function of x and is what the HIP
    kernels do.  Both are offered so the golden files can be checked against either."""
    x = _f32(x)
    s = x.max(axis=-1, keepdims=True) if shift == "max" else \
        (x.sum(axis=-1, keepdims=True, dtype=np.float32) / F32(x.shape[-1]))
    e = np.exp(x - s)
    return e / e.sum(axis=-1, keepdims=True, dtype=np.float32)


def softmax_stats(x):
    """(row max, sum of exp(x - max)) as emitted by the fused row kernel."""
    x = _f32(x)
    m = x.max(axis=-1)
    return m, np.exp(x - m[..., None]).sum(axis=-1, dtype=np.float32)


def masked_softmax(x, size, shift="max"):
    """`local_masked_softmax` with mask `j < size` (ml/primitives.spi:748-759, ml/layers.spi:409)."""
    x = _f32(x)
    mask = np.arange(x.shape[-1]) < size
    xm = np.where(mask, x, -np.inf).astype(np.float32)
    if shift == "max":
        s = xm.max(axis=-1, keepdims=True)
    else:
        s = np.where(mask, x, 0).sum(axis=-1, keepdims=True, dtype=np.float32) / F32(mask.sum())
    e = np.exp(xm - s)
    return e / e.sum(axis=-1, keepdims=True, dtype=np.float32)


def ln_l2(x):
    """`local_ln_l2` (ml/primitives.spi:701-703): x / sum(x^2), or 0 when the sum is 0."""
    x = _f32(x)
    s = (x * x).sum(axis=-1, keepdims=True, dtype=np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        return np.where(s != 0, x / s, F32(0)).astype(np.float32)


def regret_matching(x):
    """`local_regret_matching` (ml/primitives.spi:718-722)."""
    x = _f32(x)
    r = np.maximum(x, F32(0))
    s = r.sum(axis=-1, keepdims=True, dtype=np.float32)
    inv_len = F32(1) / F32(x.shape[-1])
    with np.errstate(divide="ignore", invalid="ignore"):
        return np.where(s != 0, r / s, inv_len).astype(np.float32)


def l1_normalize(x, threshold):
    """`local_l1_normalize threshold` (ml/primitives.spi:725-729): the absolute values of a row, scaled by
    threshold / sum when their sum is above the threshold (the norm is clamped, never raised)."""
    a = np.abs(_f32(x))
    s = a.sum(axis=-1, keepdims=True, dtype=np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        v = np.where(s > F32(threshold), F32(threshold) / s, F32(1)).astype(np.float32)
    return (v * a).astype(np.float32)


def reduce_all(x, op):
    """`reduce neutral f` over a whole tensor (ml/primitives.spi:136-197) for f in "+", "*", "max", "min"; integer
    sums and products wrap around like the device's."""
    x = np.asarray(x)
    flat = x.reshape(-1)
    if op in ("+", "sum"):
        return flat.sum(dtype=x.dtype) if x.dtype.kind in "iu" else flat.sum(dtype=np.float64).astype(x.dtype)
    if op in ("*", "prod"):
        return flat.prod(dtype=x.dtype) if x.dtype.kind in "iu" else flat.prod(dtype=np.float64).astype(x.dtype)
    return flat.max() if op == "max" else flat.min()


def masked_regret_matching(x, size):
    """`local_masked_regret_matching` with mask `j < size` (ml/primitives.spi:761-780)."""
    x = _f32(x)
    mask = np.arange(x.shape[-1]) < size
    r = np.where(mask, np.maximum(x, F32(0)), F32(0)).astype(np.float32)
    s = r.sum(axis=-1, keepdims=True, dtype=np.float32)
    inv_len = F32(1) / F32(mask.sum())
    with np.errstate(divide="ignore", invalid="ignore"):
        out = np.where(s != 0, r / s, inv_len)
    return np.where(mask, out, F32(0)).astype(np.float32)


def relu(x):
    """`relu = max 0` (ml/layers.spi:355)."""
    return np.maximum(_f32(x), F32(0))


# ----------------------------------------------------------------------------------------------
# scans
# ----------------------------------------------------------------------------------------------

def _lane_scan(s, t):
    """Inclusive scan of s (rows, t) over the t lanes of a row in the kernels' association."""
    r = min(t, 16)
    v = s.reshape(s.shape[0], t // r, r).copy()
    d = 1
    while d < r:
        nxt = v.copy()
        nxt[..., d:] = v[..., :-d] + v[..., d:]
        v = nxt
        d *= 2
    if t >= 32:
        v[:, 1::2, :] = v[:, 0::2, 15:16] + v[:, 1::2, :]
    if t >= 64:
        v[:, 2:4, :] = v[:, 1:2, 15:16] + v[:, 2:4, :]
    return v.reshape(s.shape[0], t)


def _wave_scan(x, inclusive=True):
    x = np.asarray(x)
    rows, cols = x.shape
    t = lanes_per_row(cols)
    chunk = 4 * t
    n_chunks = -(-cols // chunk)
    pad = n_chunks * chunk - cols
    xp = np.concatenate([x, np.zeros((rows, pad), dtype=x.dtype)], axis=1) if pad else x
    xp = xp.reshape(rows, n_chunks, t, 4)
    out = np.empty_like(xp)
    carry = np.zeros(rows, dtype=x.dtype)
    for c in range(n_chunks):
        v = xp[:, c]                                  # (rows, T, 4)
        s = ((v[..., 0] + v[..., 1]) + v[..., 2]) + v[..., 3]
        incl = _lane_scan(s, t)
        excl = np.concatenate([np.zeros((rows, 1), dtype=x.dtype), incl[:, :-1]], axis=1)
        run = carry[:, None] + excl
        for k in range(4):
            if inclusive:
                run = run + v[..., k]
                out[:, c, :, k] = run
            else:
                out[:, c, :, k] = run
                run = run + v[..., k]
        carry = carry + incl[:, -1]
    return out.reshape(rows, n_chunks * chunk)[:, :cols]


def inclusive_scan_sum(x, order="sequential"):
    """`local_inclusive_scan_sum` (ml/primitives.spi:323-325)."""
    x = np.asarray(x)
    if x.dtype.kind in "iu":
        return np.cumsum(x, axis=-1, dtype=x.dtype)
    x = _f32(x)
    if order == "sequential":
        return np.cumsum(x, axis=-1, dtype=np.float32)
    return _wave_scan(x.reshape(-1, x.shape[-1]), True).reshape(x.shape)


def exclusive_scan(x, order="sequential"):
    """`local_exclusive_scan config 0 (+)` (ml/primitives.spi:327, used on i32 in test2 :948-950)."""
    x = np.asarray(x)
    if x.dtype.kind in "iu" or order == "sequential":
        c = np.cumsum(x, axis=-1, dtype=x.dtype)
        return np.concatenate([np.zeros_like(c[..., :1]), c[..., :-1]], axis=-1)
    return _wave_scan(_f32(x).reshape(-1, x.shape[-1]), False).reshape(x.shape)


# ----------------------------------------------------------------------------------------------
# sampling
# ----------------------------------------------------------------------------------------------

def discrete_sampling(p, u, cdf=None, order="sequential"):
    """`local_discrete_sampling` (ml/primitives.spi:782-798).

    cdf = inclusive scan of p; m = max cdf over the entries with p > 0; thr = u * m (f32);
    result = the smallest j with p_j > 0 and cdf_j - thr >= 0.  `u` is one uniform in (0, 1]
    per row.  A row without any p > 0 yields INT_MAX (the reference asserts in debug builds and
    returns the reduction's neutral element otherwise).  Pass `cdf` to sample from a given
    cumulative distribution instead of recomputing it."""
    p = _f32(p)
    u = _f32(u)
    if cdf is None:
        cdf = inclusive_scan_sum(p, order)
    cdf = _f32(cdf)
    valid = p > 0
    m = np.where(valid, cdf, -np.inf).max(axis=-1)
    thr = (u * m).astype(np.float32)
    hit = valid & ((cdf - thr[..., None]).astype(np.float32) >= 0)
    j = np.arange(p.shape[-1], dtype=np.int64)
    idx = np.where(hit, j, np.int64(INT_MAX)).min(axis=-1)
    return idx.astype(np.int32)


def get_prob(p, action):
    """`local_get_prob` (ml/primitives.spi:824-830): probability of the selected action."""
    p = _f32(p)
    return np.take_along_axis(p, np.asarray(action, dtype=np.int64)[..., None], axis=-1)[..., 0]


def binarize(x, modulo):
    """`local_binarize` (ml/primitives.spi:817-821): bit j set iff not (x_j <= 0) (so a NaN sets its bit), OR-ed,
    mod `modulo`.
    The shift is the device's 32-bit shift, which gives 0 for a shift count of 32 or more (the
    source's own comment points at that difference from the CPU), so columns j >= 32 drop out.
    PARITY UNPINNED: the reference holds no output of this function."""
    x = _f32(x)
    j = np.arange(x.shape[-1], dtype=np.uint64)
    bits = np.where(~(x <= 0) & (j < 32), np.uint64(1) << (j % np.uint64(32)), np.uint64(0))
    return (np.bitwise_or.reduce(bits, axis=-1) & np.uint64(0xFFFFFFFF)) % np.uint64(modulo)


def transpose_inner(x):
    """`grid_transpose_snd` (ml/primitives.spi:36-112): swap the two innermost dimensions."""
    return np.ascontiguousarray(np.swapaxes(np.asarray(x), -1, -2))


def cem_resample(x, mask, z, noise=0.1, decay=1.0):
    """`cem` (ml/cem.spi:99-117): x (rows, ensemble) transposed weights, mask (ensemble,) winners,
    z standard normals.  winner_std = biased std * n / (n - 1) (0 for one winner); losers become
    (z * max(std, noise) + mean) * decay.  PARITY UNPINNED against the reference (it holds no
    output of this function and draws its normals on the device); pinned by closed forms."""
    x, z = _f32(x), _f32(z)
    m = np.asarray(mask).astype(bool)
    n = np.float32(m.sum())
    mean = (np.where(m, x, np.float32(0)).sum(axis=-1, dtype=np.float32) / n).astype(np.float32)
    r = (x - mean[..., None]).astype(np.float32)
    var = (np.where(m, r * r, np.float32(0)).sum(axis=-1, dtype=np.float32) / n).astype(np.float32)
    std = np.sqrt(var).astype(np.float32) * n / (n - np.float32(1)) if m.sum() > 1 else np.zeros_like(var)
    scale = np.maximum(std.astype(np.float32), np.float32(noise))
    redrawn = ((z * scale[..., None] + mean[..., None]) * np.float32(decay)).astype(np.float32)
    return np.where(m, x, redrawn).astype(np.float32)


def cem_update_rewards_mask(rewards):
    """`grid_update_rewards_mask` (ml/cem.spi:92-96): (ensemble, 2) (reward, count) pairs ->
    mask of the members whose average reward is at least the ensemble's mean (sequential f32 sum)."""
    rewards = _f32(rewards)
    r = np.where(rewards[:, 1] != 0, rewards[:, 0] / np.where(rewards[:, 1] != 0, rewards[:, 1], 1), 0).astype(np.float32)
    s = np.float32(0)
    for v in r:
        s = np.float32(s + v)
    return (r >= np.float32(s / np.float32(len(r)))).astype(np.int32)
