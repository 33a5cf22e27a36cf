"""Host surface of the row primitives (reference: ml/primitives.spi, generated ml/primitives.py).

The reference exposes `row_map`, `row_reduce` and `row_map_reduce` that run a user lambda built
from `local_*` pieces on each row (ml/primitives.spi:514-536).  A HIP library cannot take a
lambda, so every lambda the reference's tests and layers use is a named function here with the
same meaning; each one is a single fused kernel launch (libspiral_mi355.so, sp_row_*).
`main()` / `main_body()` keep the meaning of the generated module: run tests 2-6 and write the
tensors in the golden text format under test_text_outputs/primitives/.
"""
import ctypes as C
import os

import torch

from . import _console, _lib
from ._lib import PhiloxConfig, check, lib, ptr, stream_ptr

CONSTANT_SEED = 12344321            # corecuda/cupy.spi:6
THREADS_PER_BLOCK = 256             # corecuda/base.spi:14-42
BLOCKS_PER_GRID = 24


def _rows_cols(x):
    if x.dim() < 2:
        raise ValueError("expected a tensor with at least 2 dimensions")
    cols = x.shape[-1]
    return x.numel() // cols, cols


def _row_map(op, x, out=None, mask_size=0):
    rows, cols = _rows_cols(x)
    if out is None:
        out = torch.empty_like(x)
    if x.dtype == torch.float32:
        check(lib.sp_row_map_f32(op, ptr(x, name="x"), ptr(out, torch.float32, "out"), rows, cols, mask_size,
                                 stream_ptr()))
    elif x.dtype == torch.int32:
        check(lib.sp_row_map_i32(op, ptr(x, name="x"), ptr(out, torch.int32, "out"), rows, cols, stream_ptr()))
    else:
        raise TypeError("row primitives take f32 or i32 tensors, got %s" % x.dtype)
    return out


def identity(x, out=None):
    """row_map (fun config x i j_tns => x) (ml/primitives.spi:930)."""
    return _row_map(_lib.ROW_IDENTITY, x, out)


def softmax(x, out=None):
    """row_map local_softmax (ml/primitives.spi:711-716, test2 :934)."""
    return _row_map(_lib.ROW_SOFTMAX, x, out)


def masked_softmax(x, size, out=None):
    """row_map (local_masked_softmax (j < size)) (ml/primitives.spi:748-759)."""
    return _row_map(_lib.ROW_MASKED_SOFTMAX, x, out, size)


def ln_l2(x, out=None):
    """row_map local_ln_l2 (ml/primitives.spi:701-703)."""
    return _row_map(_lib.ROW_LN_L2, x, out)


def l1_normalize(x, threshold, out=None):
    """row_map (local_l1_normalize threshold) (ml/primitives.spi:725-729): |x|, scaled down to l1 norm `threshold`
    where a row's norm is above it (the decay of the average policy, ml/cfr.spi:244)."""
    rows, cols = _rows_cols(x)
    if out is None:
        out = torch.empty_like(x)
    check(lib.sp_row_l1_normalize(ptr(x, torch.float32, "x"), ptr(out, torch.float32, "out"), rows, cols, threshold,
                                  stream_ptr()))
    return out


def regret_matching(x, out=None):
    """row_map local_regret_matching (ml/primitives.spi:718-722)."""
    return _row_map(_lib.ROW_REGRET_MATCHING, x, out)


def masked_regret_matching(x, size, out=None):
    """row_map (local_masked_regret_matching (j < size)) (ml/primitives.spi:761-780)."""
    return _row_map(_lib.ROW_MASKED_REGRET_MATCHING, x, out, size)


def inclusive_scan_sum(x, out=None):
    """row_map local_inclusive_scan_sum (ml/primitives.spi:323-325); f32 or i32."""
    return _row_map(_lib.ROW_INCLUSIVE_SCAN, x, out)


def exclusive_scan_sum(x, out=None):
    """row_map (local_exclusive_scan config 0 (+)) (ml/primitives.spi:327, test2 :948-950)."""
    return _row_map(_lib.ROW_EXCLUSIVE_SCAN, x, out)


def row_ops(logits, u=None, want=("rowmax", "rowsum", "probs", "cdf", "argmax", "sample"), into=None):
    """The fused pipeline of one pass over the logits: row max, sum of exp(x - max), softmax,
    inclusive prefix sum, argmax and inverse-CDF sampling (sp_row_ops).  Returns a dict with the
    requested outputs; `into` may hold preallocated tensors for some of them."""
    rows, cols = _rows_cols(logits)
    lead = logits.shape[:-1]
    dev = logits.device
    out = {}
    for name in want:
        if into is not None and name in into:
            out[name] = into[name]
        elif name in ("probs", "cdf"):
            out[name] = torch.empty_like(logits)
        elif name in ("rowmax", "rowsum"):
            out[name] = torch.empty(lead, dtype=torch.float32, device=dev)
        elif name in ("argmax", "sample"):
            out[name] = torch.empty(lead, dtype=torch.int32, device=dev)
        else:
            raise ValueError("unknown output %r" % name)
    check(lib.sp_row_ops(ptr(logits, torch.float32, "logits"), ptr(u, torch.float32, "u"), ptr(out.get("rowmax")),
                         ptr(out.get("rowsum")), ptr(out.get("probs")), ptr(out.get("cdf")), ptr(out.get("argmax")),
                         ptr(out.get("sample")), rows, cols, 0, stream_ptr()))
    return out


def argmax(x):
    """row_reduce local_argmax (ml/primitives.spi:705-708, test2 :940); ties -> lowest index."""
    return row_ops(x, want=("argmax",))["argmax"]


def philox(mode=_lib.PHILOX_BLOCK, seed=CONSTANT_SEED, threads_per_block=THREADS_PER_BLOCK,
           blocks_per_grid=BLOCKS_PER_GRID, rows_per_block=0, offset=0, member_rows=0, member_draws=0):
    """The reference's device RNG: Philox4_32_10 seeded like `random.init {seed subsequence offset=0}`
    (ml/primitives.spi:927,1014; corecuda/random.spi:22-32).  `offset` = draws every thread's generator
    has already handed out (a graph run keeps one state per thread across its sampling nodes); member_rows /
    member_draws describe stacked runs (ensemble members evaluated in one launch), see sp_philox_t."""
    return PhiloxConfig(seed, offset, mode, threads_per_block, blocks_per_grid, rows_per_block, member_rows, member_draws)


def philox_uniforms(rng, rows, cols, out=None):
    """The uniform each of `rows` rows of width `cols` would draw from the reference's device stream `rng`."""
    if out is None:
        out = torch.empty((rows,), dtype=torch.float32, device="cuda")
    check(lib.sp_philox_uniforms(C.byref(rng), ptr(out, torch.float32, "out"), rows, cols, stream_ptr()))
    return out


def _sample(op, x, u=None, rng=None, mask_size=0, want_cdf=False, want_u=False, want_prob=False, probs_out=None,
            sample_out=None, want_probs=True):
    rows, cols = _rows_cols(x)
    probs = probs_out
    if probs is None and want_probs:
        probs = torch.empty_like(x)
    sample = torch.empty(x.shape[:-1], dtype=torch.int32, device=x.device) if sample_out is None else sample_out
    cdf = torch.empty_like(x) if want_cdf else None
    u_out = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device) if want_u else None
    prob = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device) if want_prob else None
    if (u is None) == (rng is None):
        raise ValueError("give exactly one of u (a tensor of uniforms in (0, 1]) and rng (a PhiloxConfig)")
    if (probs is not None and probs.shape != x.shape) or sample.shape != x.shape[:-1]:
        raise ValueError("the output tensors do not have the input's dimensions")
    check(lib.sp_row_sample(op, ptr(x, torch.float32, "x"), ptr(u, torch.float32, "u"),
                            C.byref(rng) if rng is not None else None,
                            ptr(probs, torch.float32, "probs") if probs is not None else None, ptr(cdf),
                            ptr(u_out), ptr(sample, torch.int32, "sample"), ptr(prob), rows, cols, mask_size,
                            stream_ptr()))
    res = (probs, sample)
    if want_cdf:
        res += (cdf,)
    if want_u:
        res += (u_out,)
    if want_prob:
        res += (prob,)
    return res


def discrete_sampling(p, u=None, rng=None, **kw):
    """row_reduce local_discrete_sampling (ml/primitives.spi:782-798)."""
    return _sample(_lib.ROW_IDENTITY, p, u, rng, **kw)


def softmax_and_discrete_sampling(x, u=None, rng=None, **kw):
    """row_map_reduce local_softmax_and_discrete_sampling (ml/primitives.spi:800-802)."""
    return _sample(_lib.ROW_SOFTMAX, x, u, rng, **kw)


def masked_softmax_and_discrete_sampling(x, size, u=None, rng=None, **kw):
    """row_map_reduce local_masked_softmax_and_discrete_sampling (ml/primitives.spi:804-806)."""
    return _sample(_lib.ROW_MASKED_SOFTMAX, x, u, rng, mask_size=size, **kw)


def regret_matching_and_discrete_sampling(x, u=None, rng=None, **kw):
    """row_map_reduce local_regret_matching_and_discrete_sampling (ml/primitives.spi:808-810)."""
    return _sample(_lib.ROW_REGRET_MATCHING, x, u, rng, **kw)


def masked_regret_matching_and_discrete_sampling(x, size, u=None, rng=None, **kw):
    """row_map_reduce local_masked_regret_matching_and_discrete_sampling (ml/primitives.spi:812-814)."""
    return _sample(_lib.ROW_MASKED_REGRET_MATCHING, x, u, rng, mask_size=size, **kw)


_ROW_OPS = {"identity": _lib.ROW_IDENTITY, "softmax": _lib.ROW_SOFTMAX, "masked_softmax": _lib.ROW_MASKED_SOFTMAX,
            "ln_l2": _lib.ROW_LN_L2, "regret_matching": _lib.ROW_REGRET_MATCHING,
            "masked_regret_matching": _lib.ROW_MASKED_REGRET_MATCHING}


def get_prob(x, action_id, op="identity", size=0):
    """row_gather_reduce of `local_get_prob config action_id (zip probs j_tns)` (ml/primitives.spi:824-830):
    the value of op(x) at column action_id[r] of every row, e.g. `get_policy_probs` of the CFR agent with
    op="masked_regret_matching" (ml/cfr.spi:97-107)."""
    rows, cols = _rows_cols(x)
    if action_id.shape != x.shape[:-1]:
        raise ValueError("one action id per row expected")
    out = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    check(lib.sp_row_get_prob(_ROW_OPS[op], ptr(x, torch.float32, "x"), ptr(action_id, torch.int32, "action_id"),
                              ptr(out), rows, cols, size, stream_ptr()))
    return out


def get_action(x, u=None, rng=None, op="identity", size=0):
    """The agents' `get_action` (ml/cem.spi:152-164, ml/cfr.spi:117-129): row_gather_reduce of a discrete
    sample from op(x) together with the probability it was drawn with.  With `rng` the default stream is the
    gather mapping (one row per thread).  Returns (prob, action_id)."""
    if u is None and rng is None:
        rng = philox(_lib.PHILOX_GATHER)
    _, action, prob = _sample(_ROW_OPS[op], x, u, rng, mask_size=size, want_prob=True, want_probs=False)
    return prob, action


def binarize(x, modulo, out=None):
    """row_reduce local_binarize (ml/primitives.spi:817-821; layer head ml/layers.spi:439-446)."""
    rows, cols = _rows_cols(x)
    if out is None:
        out = torch.empty(x.shape[:-1], dtype=torch.int32, device=x.device)   # holds the reference's u32
    check(lib.sp_row_binarize(ptr(x, torch.float32, "x"), ptr(out, torch.int32, "out"), rows, cols, modulo,
                              stream_ptr()))
    return out


def cem_update_rewards_mask(rewards, mask=None):
    """`grid_update_rewards_mask` (ml/cem.spi:92-96): rewards (ensemble, 2) f32 (reward sum, count) pairs are
    turned into the winners' mask (average reward at or above the ensemble's mean) and zeroed."""
    if rewards.dim() != 2 or rewards.shape[1] != 2:
        raise ValueError("rewards must be (ensemble, 2)")
    n = rewards.shape[0]
    if mask is None:
        mask = torch.empty((n,), dtype=torch.int32, device=rewards.device)
    check(lib.sp_cem_update_mask(ptr(rewards, torch.float32, "rewards"), ptr(mask, torch.int32, "mask"), n, stream_ptr()))
    return mask


def cem(transposed_weights, mask, normals=None, noise=0.1, decay=1.0, out=None, generator=None, rng=None):
    """`cem rng transposed_weights model` (ml/cem.spi:99-117), in place by default like the reference:
    every row holds one weight position across the ensemble; the members outside `mask` are redrawn from the
    winners' mean and spread.  `rng=(seed, offset)` draws the normals on the device like the reference does
    (curand_normal on Philox4_32_10, row r = subsequence r, `offset` draws in; sp_cem_resample_philox); otherwise
    `normals` (same shape) is used, which defaults to fresh standard normals from torch."""
    rows, cols = _rows_cols(transposed_weights)
    if mask.shape != (cols,):
        raise ValueError("one mask entry per ensemble member expected")
    if out is None:
        out = transposed_weights
    if rng is not None:
        if normals is not None:
            raise ValueError("give normals or rng, not both")
        seed, offset = rng
        check(lib.sp_cem_resample_philox(ptr(transposed_weights, torch.float32, "transposed_weights"),
                                         ptr(mask, torch.int32, "mask"), seed, offset, ptr(out, torch.float32, "out"),
                                         rows, cols, noise, decay, stream_ptr()))
        return out
    if normals is None:
        normals = torch.randn(transposed_weights.shape, generator=generator, device=transposed_weights.device,
                              dtype=torch.float32)
    check(lib.sp_cem_resample(ptr(transposed_weights, torch.float32, "transposed_weights"), ptr(mask, torch.int32, "mask"),
                              ptr(normals, torch.float32, "normals"), ptr(out, torch.float32, "out"), rows, cols, noise,
                              decay, stream_ptr()))
    return out


_REDUCE_OPS = {"sum": _lib.REDUCE_SUM, "+": _lib.REDUCE_SUM, "prod": _lib.REDUCE_PROD, "*": _lib.REDUCE_PROD,
               "max": _lib.REDUCE_MAX, "min": _lib.REDUCE_MIN, "average": _lib.REDUCE_AVERAGE}
_MAP_IN = {"identity": _lib.MAP_IN_IDENTITY, "id": _lib.MAP_IN_IDENTITY, "square": _lib.MAP_IN_SQUARE,
           "sqr": _lib.MAP_IN_SQUARE, "abs": _lib.MAP_IN_ABS}
_MAP_OUT = {"identity": _lib.MAP_OUT_IDENTITY, "id": _lib.MAP_OUT_IDENTITY, "sqrt": _lib.MAP_OUT_SQRT}


def row_reduce(x, op="sum", map_in="identity", map_out="identity", out=None):
    """One reduction along the innermost dimension: out[...] = map_out(reduce_j map_in(x[..., j])) (sp_row_reduce_f32).
    `row_reduce` of the `local_*` reductions (ml/primitives.spi:330-348,523-526) and `reduce_2d` /
    `map_reduce_map_2d` (:593-660); the inner dimension may be any multiple of 4."""
    rows, cols = _rows_cols(x) if x.dim() >= 2 else (1, x.numel())
    if out is None:
        out = torch.empty(x.shape[:-1] if x.dim() >= 2 else (1,), dtype=torch.float32, device=x.device)
    if out.numel() != rows:
        raise ValueError("The first dimension of the input has to equal the dimension of the output in the reduce_2d kernel.")
    check(lib.sp_row_reduce_f32(_REDUCE_OPS[op], _MAP_IN[map_in], _MAP_OUT[map_out], ptr(x, torch.float32, "x"),
                                ptr(out, torch.float32, "out"), rows, cols, stream_ptr()))
    return out


def local_sum(x):
    """row_reduce local_sum (ml/primitives.spi:338)."""
    return row_reduce(x, "sum")


def local_prod(x):
    """row_reduce local_prod (ml/primitives.spi:344)."""
    return row_reduce(x, "prod")


def local_max(x):
    """row_reduce local_max (ml/primitives.spi:346)."""
    return row_reduce(x, "max")


def local_min(x):
    """row_reduce local_min (ml/primitives.spi:348)."""
    return row_reduce(x, "min")


def local_average(x):
    """row_reduce local_average (ml/primitives.spi:342): local_sum / local_length."""
    return row_reduce(x, "average")


def local_length(x):
    """local_length (ml/primitives.spi:340): the extent of the innermost dimension."""
    return x.shape[-1]


def map_reduce_map_2d(map_in, neutral_element, f, map_out, from_, to=None):
    """`map_reduce_map_2d map_in neutral_element f map_out from to` (ml/primitives.spi:647-651) for the named
    lambdas: map_in in {"id", "sqr", "abs"}, f in {"+", "*", "max", "min"} with its own neutral element (the
    argument is checked against it), map_out in {"id", "sqrt"}.  `map_reduce_map_2d("sqr", 0, "+", "sqrt", w_t)`
    is the per-row weight norm of the CEM update (ml/cem.spi:139)."""
    neutral = {"+": 0.0, "sum": 0.0, "*": 1.0, "prod": 1.0, "max": float("-inf"), "min": float("inf")}[f]
    if float(neutral_element) != neutral and not (f == "max" and float(neutral_element) == 0.0 and map_in in ("sqr", "square", "abs")):
        raise ValueError("the neutral element of %r is %r" % (f, neutral))
    return row_reduce(from_, f, map_in, map_out, out=to)


grid_map_reduce_map_2d = map_reduce_map_2d


def reduce_2d(neutral_element, f, from_, to=None):
    """`reduce_2d neutral_element f from to` (ml/primitives.spi:617-618)."""
    return map_reduce_map_2d("id", neutral_element, f, "id", from_, to)


def reduce_max(x):
    """`grid_reduce grid 0 max norms` of the CEM update's weight-norm print (ml/cem.spi:140): the largest element of a
    tensor, as a 0-d tensor; one launch over the whole device (sp_reduce)."""
    return reduce("max", x)


def reduce_min(x):
    """`reduce limit.max min` over a whole tensor (ml/primitives.spi:176-197)."""
    return reduce("min", x)


def grid_transpose(x, out=None):
    """`grid_transpose from to` (ml/primitives.spi:100-112): 2-D transpose, e.g. (ensemble, dim) <-> (dim, ensemble)
    of the CEM weight duals (ml/cem.spi:131-146)."""
    return transpose_snd(x, out)


def map(op, x, out=None):  # noqa: A001  (the reference's name, ml/primitives.spi:128)
    """primitives.map f from to for f in {"copy", "relu", "tanh", "sigmoid"} (ml/layers.spi:353-355)."""
    code = {"copy": _lib.MAP_COPY, "relu": _lib.MAP_RELU, "tanh": _lib.MAP_TANH, "sigmoid": _lib.MAP_SIGMOID}[op]
    if out is None:
        out = torch.empty_like(x)
    check(lib.sp_map_f32(code, ptr(x, torch.float32, "x"), ptr(out, torch.float32, "out"), x.numel(), stream_ptr()))
    return out


_workspace = {}


def _reduce_workspace(device):
    key = device.index
    if key not in _workspace:
        # zero-filled once: the give-up counter behind the blocks' slots starts from what it finds
        _workspace[key] = torch.zeros(lib.sp_reduce_workspace_bytes(), dtype=torch.uint8, device=device)
    return _workspace[key]


def reduce(f, x):  # noqa: A001  (the reference's name, ml/primitives.spi:176)
    """`reduce neutral f` / `grid_reduce grid neutral f` over a whole tensor (ml/primitives.spi:136-197) for f in
    {"+", "*", "max", "min"} with its own neutral element.  f32, i32 or u64 (carried as int64 by torch).  Returns a
    0-d tensor on the device."""
    op = {"+": _lib.REDUCE_SUM, "sum": _lib.REDUCE_SUM, "*": _lib.REDUCE_PROD, "prod": _lib.REDUCE_PROD,
          "max": _lib.REDUCE_MAX, "min": _lib.REDUCE_MIN}[f]
    code = {torch.float32: 0, torch.int32: 1, torch.int64: 2}[x.dtype]
    ws = _reduce_workspace(x.device)
    out = torch.empty(4, dtype=x.dtype, device=x.device)  # 16-byte aligned scalar slot
    check(lib.sp_reduce(op, code, ptr(x, name="x"), ptr(out), x.numel(), ptr(ws), ws.numel(), stream_ptr()))
    return out[0]


grid_reduce = reduce


def reduce_sum(x):
    """reduce 0 (+) / grid_reduce grid 0 (+) over a whole tensor (ml/primitives.spi:176-197)."""
    return reduce("+", x)


def reduce_give_ups(device=None):
    """How often a reduce on this device's workspace gave up waiting for its partial results (sp_reduce_status; waits
    for the current stream).  0 unless other work kept part of a launch off the device for milliseconds."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    ws = _reduce_workspace(dev)
    n = C.c_int64(0)
    check(lib.sp_reduce_status(ptr(ws), ws.numel(), C.byref(n), stream_ptr()))
    return n.value


def reduce_sum_static(x, out):
    """reduce_sum without any allocation: the scratch memory is an array inside the library (sp_reduce_sum_static),
    the result goes to out[0] of a caller-owned, 16-byte aligned tensor of x's dtype.  Calls on one GPU must not
    overlap in time."""
    code = {torch.float32: 0, torch.int32: 1, torch.int64: 2}[x.dtype]
    check(lib.sp_reduce_sum_static(code, ptr(x, name="x"), ptr(out, x.dtype, "out"), x.numel(), stream_ptr()))
    return out


def transpose_snd(x, out=None):
    """grid_transpose_snd from to: swap the two innermost dimensions (ml/primitives.spi:107-109)."""
    if x.element_size() != 4 or x.dim() < 2:
        raise TypeError("transpose_snd takes tensors of 4-byte elements with >= 2 dimensions")
    b, c = x.shape[-2], x.shape[-1]
    a = x.numel() // (b * c)
    if out is None:
        out = torch.empty(x.shape[:-2] + (c, b), dtype=x.dtype, device=x.device)
    check(lib.sp_transpose_inner_b32(ptr(x, name="x"), ptr(out, name="out"), a, b, c, stream_ptr()))
    return out


# ----------------------------------------------------------------------------------------------
# self-tests in the reference's format
# ----------------------------------------------------------------------------------------------

def _dump(root, head_dir, name, limit, *tensors):
    d = os.path.join(root, head_dir)
    os.makedirs(d, exist_ok=True)
    _console.write_ln(os.path.join(d, name), limit, *[t.cpu().numpy() for t in tensors])


def _row_test(root, m, n, head_dir, grid, seed=CONSTANT_SEED):
    """ml/primitives.spi test2 (:904-988, block level) and test4 (:992-1076, grid level).  They differ
    in which Philox subsequence a row uses and in test2 overwriting output_softmax'.txt."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    ident = torch.arange(m * n, dtype=torch.int32, device="cuda").reshape(m, n)
    x = torch.randn((m, n), generator=gen, device="cuda", dtype=torch.float32)
    rng = philox(_lib.PHILOX_GRID if grid else _lib.PHILOX_BLOCK)
    ii = torch.arange(m, dtype=torch.int32, device="cuda")[:, None].expand(m, n)
    jj = torch.arange(n, dtype=torch.int32, device="cuda")[None, :].expand(m, n)
    sm = softmax(x)
    probs1, sample1 = softmax_and_discrete_sampling(x, rng=rng)
    probs2, sample2 = masked_softmax_and_discrete_sampling(x, 11, rng=rng)
    if not grid:
        _dump(root, head_dir, "output_reduce.txt", 1024, reduce_sum(x))
    _dump(root, head_dir, "input.txt", 1024, x)
    _dump(root, head_dir, "input_identity.txt", 1024, ident)
    _dump(root, head_dir, "output_softmax.txt", 1024, sm)
    _dump(root, head_dir, "output_masked_softmax.txt", 1024, masked_softmax(x, 4))
    _dump(root, head_dir, "output_ln.txt", 1024, ln_l2(x))
    _dump(root, head_dir, "output_argmax.txt", 1024, argmax(x))
    _dump(root, head_dir, "output_softmax_scan.txt", m * n, sm, inclusive_scan_sum(sm))
    _dump(root, head_dir, "output_identity.txt", m * n, identity(ident))
    _dump(root, head_dir, "output_indices_map.txt", m * n, ii, jj)
    _dump(root, head_dir, "output_indices_reduction.txt", m * n, ii[:, 0])
    _dump(root, head_dir, "output_sum_exclusive.txt", m * n, exclusive_scan_sum(ident))
    _dump(root, head_dir, "output_softmax'.txt", 1024, probs1)
    _dump(root, head_dir, "output_sampling.txt", 1024, sample1)
    _dump(root, head_dir, "output_softmax'.txt" if not grid else "output_softmax''.txt", 1024, probs2)
    _dump(root, head_dir, "output_sampling'.txt", 1024, sample2)


def test2(m, n, head_dir, root="test_text_outputs/primitives/"):
    _row_test(root, m, n, head_dir, grid=False)


def test3(n, head_dir, root="test_text_outputs/primitives/"):
    """ml/primitives.spi test3 (:851-902): the `row_gather_*` ops, one row of width n per thread of the grid
    (threads_per_block * blocks_per_grid rows).  Row indices, the identity map, masked (j < 3) regret matching
    and a masked-softmax sample drawn from each thread's own Philox subsequence."""
    m = THREADS_PER_BLOCK * BLOCKS_PER_GRID
    gen = torch.Generator(device="cuda")
    gen.manual_seed(CONSTANT_SEED)
    input_identity = torch.arange(m * n, dtype=torch.float32, device="cuda").reshape(m, n)
    x = torch.randn((m, n), generator=gen, device="cuda", dtype=torch.float32)
    ii = torch.arange(m, dtype=torch.int32, device="cuda")[:, None].expand(m, n)
    jj = torch.arange(n, dtype=torch.int32, device="cuda")[None, :].expand(m, n)
    _, sample = masked_softmax_and_discrete_sampling(x, 3, rng=philox(_lib.PHILOX_GATHER), want_probs=False)
    _dump(root, head_dir, "input_identity.txt", 1024, input_identity)
    _dump(root, head_dir, "output_sample_reduce.txt", 1024, sample)
    _dump(root, head_dir, "output_indices_map.txt", 1024, ii, jj)
    _dump(root, head_dir, "output_indices_reduce.txt", 1024, ii[:, 0])
    _dump(root, head_dir, "output_op_map.txt", 1024, masked_regret_matching(x, 3))
    _dump(root, head_dir, "zip_input_output_identity_map.txt", 1024, x, identity(x))


def test4(m, n, head_dir, root="test_text_outputs/primitives/"):
    _row_test(root, m, n, head_dir, grid=True)


def test5(l, m, n, head_dir, root="test_text_outputs/primitives/"):
    """ml/primitives.spi test5 (:1078-1088): transpose of arange(l, m, n)."""
    x = torch.arange(l * m * n, dtype=torch.int32, device="cuda").reshape(l, m, n)
    y = transpose_snd(x)
    d = os.path.join(root, head_dir)
    os.makedirs(d, exist_ok=True)
    with open(os.path.join(d, "transpose.txt"), "w") as f:
        f.write(_console.format_tensor(2 ** 31 - 1, x.cpu().numpy()) + "\n")
        f.write(_console.format_tensor(2 ** 31 - 1, y.cpu().numpy()) + "\n")


def test6(m, n, head_dir, root="test_text_outputs/primitives/"):
    """ml/primitives.spi test6 (:1090-1110): u64 sum of arange(m * n), block and grid variants."""
    x = torch.arange(m * n, dtype=torch.int64, device="cuda").reshape(m, n)
    r = reduce_sum(x)
    _dump(root, head_dir, "input_identity.txt", 1024, x)
    _dump(root, head_dir, "output_reduce_block.txt", 1024, r)
    _dump(root, head_dir, "output_reduce_grid.txt", 1024, r)


def main_body(root="test_text_outputs/primitives/"):
    """ml/primitives.spi main (:1112-1137): tests 2 to 6 in the reference's order."""
    test2(1 << 6, 1 << 7, "test2/a/", root)
    test2(1 << 7, 1 << 6, "test2/b/", root)
    test3(1 << 4, "test3/a", root)
    test3(1 << 8, "test3/b", root)
    test4(1 << 7, 1 << 6, "test4/b/", root)
    test4(1 << 6, 1 << 7, "test4/a/", root)
    test5(2, 4, 8, "test5/a", root)
    test5(2, 128, 256, "test5/b", root)
    test6(128, 128, "test6/a", root)


def main():
    main_body()
    torch.cuda.current_stream().synchronize()
    print("Done.")


if __name__ == "__main__":
    main()
