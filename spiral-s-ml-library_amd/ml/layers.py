"""Host surface of the dense layers (reference: ml/layers.spi, generated ml/layers.py).

Two levels:

* `mlp_forward`: a dense stack with ReLU between layers and a row head as ONE fused kernel
  (sp_mlp_forward); activations never leave the compute unit.
* the reference's static layer graph (ml/layers.spi:24-55): the same node constructors
  (`input`, `weight`, `matmul`, `matmul_ensemble`, `tanh`/`sigmoid`/`relu`, `ln_l2`, `softmax`,
  `regret_matching`, `argmax`, `discrete_sample`, `softmax_and_discrete_sample`, `masked_*`,
  `binarize`, `copy`, `pair`, `apply`, `key_graph`), the same byte-arena layout (`create_model`,
  `pass_calculate_partitions`: three arenas -- weights, workspace, weight adjoints -- every tensor at
  a 16-byte aligned offset in depth-first order, :127-179 and corebase/partitionm.spi:53-67) so a
  `model_ptrs` triple can be exchanged with code that lays the arenas out like the reference, and
  `graph_run_host`, which runs every node through the C ABI.  The reference interprets the graph
  inside one kernel (:181-252); here each node is one library call on the caller's stream, and a
  relu-MLP with a sampling head collapses into the fused kernel when its shapes allow.

A primed constructor of the reference (`softmax' out x`) is the underscore form here with a graph
for `out` (`softmax_(out, x)`); every constructor also curries on its last argument so that
`pipe(input(...), matmul((64, 64)), ln_l2, relu)` reads like the reference's `|>` chains.
"""
import builtins
import ctypes as C
import itertools

import torch

from . import _console, _lib, matmul as _matmul, primitives as _prim
from ._lib import check, lib, ptr, stream_ptr

HEADS = {None: _lib.HEAD_NONE, "none": _lib.HEAD_NONE, "softmax": _lib.HEAD_SOFTMAX,
         "regret_matching": _lib.HEAD_REGRET_MATCHING, "softmax_regret_matching": _lib.HEAD_SOFTMAX_RM}


# ----------------------------------------------------------------------------------------------
# fused dense stack
# ----------------------------------------------------------------------------------------------

class PackedWeights:
    """The weights of a dense stack in the order the packed kernel multiplies them in (sp_mlp_pack_weights):
    `buffer` is one uint8 tensor, `dims` the layer widths, `dtype` the storage type.  A snapshot: pack again after
    the weights have changed (`pack_weights(weights, into=packed)` reuses the buffer)."""

    def __init__(self, buffer, dims, dtype):
        self.buffer, self.dims, self.dtype = buffer, list(dims), dtype


def packed_bytes(dims):
    """Bytes of the packed form of a stack with these widths; 0 when the packed kernel does not take the stack."""
    return int(lib.sp_mlp_packed_bytes(len(dims) - 1, (C.c_int32 * len(dims))(*dims)))


def pack_weights(weights, into=None):
    """Pack the row-major weights [(out_i, in_i), ...] of a stack once, for `mlp_forward(..., packed=...)`.
    Returns None when the packed kernel does not take the stack (then call mlp_forward with the weights)."""
    dims = [weights[0].shape[1]] + [w.shape[0] for w in weights]
    need = packed_bytes(dims)
    if need == 0:
        return None
    n = len(weights)
    if into is None:
        into = PackedWeights(torch.empty(need, dtype=torch.uint8, device=weights[0].device), dims, weights[0].dtype)
    elif into.dims != dims or into.dtype != weights[0].dtype:
        raise ValueError("the packed buffer was made for another stack")
    wp = (C.c_void_p * n)(*[ptr(w, weights[0].dtype, "weights[%d]" % i) for i, w in enumerate(weights)])
    check(lib.sp_mlp_pack_weights(_lib.DTYPES[weights[0].dtype], n, wp, (C.c_int32 * (n + 1))(*dims), ptr(into.buffer),
                                  into.buffer.numel(), stream_ptr()))
    return into


def mlp_forward(x, weights, biases=None, head="softmax_regret_matching", u=None, mask_size=0, want_logits=False,
                policy_out=None, action_out=None, packed=None, rng=None):
    """policy, action[, logits] = fused forward of relu-MLP + head + discrete sampling.

    x: (batch, in) f16/bf16; weights[i]: (out_i, in_i) of the same dtype (the B operand of A.B^T,
    ml/layers.spi:227-240,467); biases: optional list of f32 (out_i,) or None entries (build
    extension, the reference has no bias); u: (batch,) f32 uniforms in (0, 1] or None (no action).
    head: None | "softmax" | "regret_matching" | "softmax_regret_matching"; mask_size > 0 restricts
    the head to columns j < mask_size (masked_* layers, ml/layers.spi:408-432).  packed: the result of
    pack_weights(weights) -- the stack then runs on the packed kernel and `weights` is not read.  rng: instead of
    u, a Philox stream (primitives.philox(...)) the head draws its uniforms from inside the kernel, row r taking
    what primitives.philox_uniforms(rng, batch, out) hands out for it (ml/layers.spi:339-344)."""
    if packed is not None:
        n, dims = len(packed.dims) - 1, packed.dims
        if packed.dtype != x.dtype:
            raise TypeError("the packed weights must have the dtype of x")
        assert x.shape[1] == dims[0], "The K dimension of the A and B tensors must match."
    else:
        n = len(weights)
        dims = [x.shape[1]] + [w.shape[0] for w in weights]
        for i, w in enumerate(weights):
            if w.dtype != x.dtype:
                raise TypeError("weights[%d] must have the dtype of x" % i)
            assert w.shape[1] == dims[i], "The K dimension of the A and B tensors must match."
    batch = x.shape[0]
    policy = policy_out if policy_out is not None else \
        torch.empty((batch, dims[-1]), dtype=torch.float32, device=x.device)
    action = action_out
    if action is None and (u is not None or rng is not None):
        action = torch.empty((batch,), dtype=torch.int32, device=x.device)
    logits = torch.empty((batch, dims[-1]), dtype=torch.float32, device=x.device) if want_logits else None
    bp = None
    if biases is not None:
        bp = (C.c_void_p * n)(*[ptr(b, torch.float32, "biases[%d]" % i) if b is not None else None
                                for i, b in enumerate(biases)])
    dp = (C.c_int32 * (n + 1))(*dims)
    if packed is not None:
        check(lib.sp_mlp_forward_packed(_lib.DTYPES[x.dtype], ptr(x, name="x"), n, ptr(packed.buffer),
                                        packed.buffer.numel(), bp, dp, ptr(u, torch.float32, "u"),
                                        C.byref(rng) if rng is not None else None, ptr(policy, torch.float32, "policy_out"),
                                        ptr(action, torch.int32, "action_out"), ptr(logits), batch, HEADS[head],
                                        mask_size, stream_ptr()))
    else:
        wp = (C.c_void_p * n)(*[ptr(w, name="weights[%d]" % i) for i, w in enumerate(weights)])
        check(lib.sp_mlp_forward(_lib.DTYPES[x.dtype], ptr(x, name="x"), n, wp, bp, dp, ptr(u, torch.float32, "u"),
                                 C.byref(rng) if rng is not None else None, ptr(policy, torch.float32, "policy_out"), ptr(action, torch.int32, "action_out"),
                                 ptr(logits), batch, HEADS[head], mask_size, stream_ptr()))
    out = (policy, action)
    return out + (logits,) if want_logits else out


def mlp_forward_ensemble(x, weights, head="regret_matching", u=None, mask_size=0, policy_out=None, action_out=None,
                         rng=None):
    """policy[, action] of every member of an ensemble of one- or two-layer f32 stacks on one shared input, one launch:
    policy[e] = head(relu(x . weights[0][e]^T) . weights[1][e]^T), or head(x . weights[0][e]^T) for a single layer.

    x: (batch, in) f32; two layers: weights[0]: (E, 64, in), weights[1]: (E, out, 64), in a multiple of 8 up to 128;
    one layer: weights[0]: (E, out, in), in a multiple of 8 up to 256 (the tensors of `matmul_ensemble`,
    ml/layers.spi:468-479); head and mask_size as for mlp_forward, with at most 4 computed outputs (out, or mask_size).
    u: (E, batch) uniforms or rng: a Philox stream over the E * batch stacked rows (member_rows = batch) for an action
    per member and row; without either only the policy (E, batch, out) is computed -- the graphs of the reference's CEM
    policies, game/leduc/model_cem.spi:55-63 and game/nl_hu_holdem/model_cem.spi:84-100."""
    n = len(weights)
    if n not in (1, 2):
        raise ValueError("one weight tensor (E, out, in), or two: (E, 64, in) and (E, out, 64)")
    if x.dtype != torch.float32 or any(w.dtype != torch.float32 for w in weights):
        raise TypeError("x and the weights must be f32")
    members, batch = weights[0].shape[0], x.shape[0]
    assert all(w.shape[0] == members for w in weights), "every layer needs one matrix per member"
    dims = [x.shape[1]] + [w.shape[1] for w in weights]
    for i, w in enumerate(weights):
        assert w.shape[2] == dims[i], "The K dimension of the A and B tensors must match."
    policy = policy_out if policy_out is not None else \
        torch.empty((members, batch, dims[-1]), dtype=torch.float32, device=x.device)
    action = action_out
    if action is None and (u is not None or rng is not None):
        action = torch.empty((members, batch), dtype=torch.int32, device=x.device)
    wp = (C.c_void_p * n)(*[ptr(w, name="weights[%d]" % i) for i, w in enumerate(weights)])
    dp = (C.c_int32 * (n + 1))(*dims)
    check(lib.sp_mlp_forward_ensemble(_lib.SP_F32, ptr(x, name="x"), n, wp, dp, members, ptr(u, torch.float32, "u"),
                                      C.byref(rng) if rng is not None else None, ptr(policy, torch.float32, "policy_out"),
                                      ptr(action, torch.int32, "action_out"), batch, HEADS[head], mask_size, stream_ptr()))
    return (policy, action) if action is not None else policy


def ensemble_binarize(x, weights, modulo, out=None):
    """out[e][r] = binarize(x[r] . weights[e]^T) mod modulo for every member of an ensemble layer, one launch, the
    product never written: the graph of the reference's CFR models (`matmul_ensemble -> binarize'`,
    game/leduc/model_cfr.spi:56-61; ml/primitives.spi:817-821).  x: (batch, in) f32, in a multiple of 8 up to 256;
    weights: (E, out, in) f32; out: (E, batch) i32 holding the u32 words."""
    if x.dtype != torch.float32 or weights.dtype != torch.float32:
        raise TypeError("x and the weights must be f32")
    members, n, k0 = weights.shape
    assert k0 == x.shape[1], "The K dimension of the A and B tensors must match."
    if out is None:
        out = torch.empty((members, x.shape[0]), dtype=torch.int32, device=x.device)
    check(lib.sp_ensemble_binarize(_lib.SP_F32, ptr(x, name="x"), ptr(weights, name="weights"), ptr(out, torch.int32, "out"),
                                   members, x.shape[0], k0, n, modulo, stream_ptr()))
    return out


# ----------------------------------------------------------------------------------------------
# the layer graph (ml/layers.spi:6-55)
# ----------------------------------------------------------------------------------------------

def weight_id():
    return 0


def workspace_id():
    """For input layers and intermediates."""
    return 1


def weight_adjoint_id():
    return 2


def num_spaces():
    return 3


THREADS_PER_BLOCK = 256
_blocks_per_grid = None
_generator = {}

DTYPES = {"float": torch.float32, "f32": torch.float32, "int": torch.int32, "i32": torch.int32,
          "uint": torch.int32,   # u32 bit patterns; torch has no arithmetic-free u32 views on all builds
          "f16": torch.float16, "bf16": torch.bfloat16}


def _dtype(t):
    return DTYPES[t] if isinstance(t, str) else t


def blocks_per_grid():
    """The leading dimension every workspace tensor of a graph must have (ml/layers.spi:81-106).  In
    the reference it is the number of SMs, because block b of its one kernel owns slice b; here it
    is a free batch split, by default the number of compute units."""
    global _blocks_per_grid
    if _blocks_per_grid is None:
        _blocks_per_grid = _lib.device_info()["compute_units"] if torch.cuda.is_available() else 24
    return _blocks_per_grid


def set_blocks_per_grid(n):
    global _blocks_per_grid
    _blocks_per_grid = int(n)


def set_random_seed(seed=_prim.CONSTANT_SEED, device="cuda"):
    """`cupy.set_random_seed` (corecuda/cupy.spi:9): reseeds the generator the initialisers draw from."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    _generator[torch.device(device).type] = g
    return g


def _gen(device):
    key = torch.device(device).type
    return _generator[key] if key in _generator else set_random_seed(device=device)


class TensorSpec:
    """Dimensions and element type of one tensor: the `D_D dim` leaf of `dim_of` (ml/layers.spi:56-58)."""
    __slots__ = ("dim", "dtype")

    def __init__(self, dim, dtype):
        self.dim, self.dtype = tuple(int(d) for d in dim), dtype

    def __eq__(self, o):
        return isinstance(o, TensorSpec) and self.dim == o.dim

    def __repr__(self):
        return "TensorSpec(%r, %s)" % (self.dim, self.dtype)

    @property
    def nbytes(self):
        n = 1
        for d in self.dim:
            n *= d
        return n * torch.empty((), dtype=self.dtype).element_size()


class Graph:
    """Base of the node types of `union rec graph t` (ml/layers.spi:24-55).  Nodes compare by identity."""


class Layer(Graph):
    def __init__(self, space_id, dim, init=None, dtype="float"):
        self.space_id, self.spec, self.init = space_id, TensorSpec(dim, _dtype(dtype)), init


class KeyGraph(Graph):
    def __init__(self, key, x):
        self.key, self.x = key, x


class KeyScalar(Graph):
    def __init__(self, key):
        self.key = key


class Apply(Graph):
    def __init__(self, a, b):
        self.a, self.b = a, b


class Pair(Graph):
    def __init__(self, a, b):
        self.a, self.b = a, b


class Zip(Graph):
    def __init__(self, a, b):
        self.a, self.b = a, b


class Fst(Graph):
    def __init__(self, x):
        self.x = x


class Snd(Graph):
    def __init__(self, x):
        self.x = x


class BlockMap(Graph):
    def __init__(self, f, a, out=None):
        self.f, self.a, self.out = f, a, out


class BlockRowMap(Graph):
    def __init__(self, f, a, out=None, size=0):
        self.f, self.a, self.out, self.size = f, a, out, size


class BlockRowReduce(Graph):
    def __init__(self, f, a, out=None, arg=0):
        self.f, self.a, self.out, self.arg = f, a, out, arg


class BlockRowMapReduce(Graph):
    def __init__(self, f, a, out=None, size=0):
        self.f, self.a, self.out, self.size = f, a, out, size


class BlockMatmul(Graph):
    def __init__(self, a, b):
        self.a, self.b = a, b


_REDUCE_DTYPE = {"argmax": torch.int32, "discrete_sample": torch.int32, "binarize": torch.int32, "max": None}


def _row_dtype(t):
    return torch.float32 if t in (torch.float16, torch.bfloat16) else t


def get_dim_pair(h, x):
    """Top-level dimensions of a node, memoised in `h` (ml/layers.spi:75-125): a TensorSpec or a pair of
    them.  The asserts are the reference's."""
    if x in h:
        return h[x]
    q_msg = "The batch dimension in the %s node needs to equal the number of blocks per grid."

    def check_out(spec, out):
        if out is not None:
            assert spec == get_dim_pair(h, out), \
                "The dimensions coming from the input and the dimensions of the output have to match."

    if isinstance(x, BlockRowMapReduce):
        a = get_dim(h, x.a)
        q, w, e = a.dim
        assert q == blocks_per_grid(), q_msg % "row reduce"
        # the row heads compute and store f32 whatever the stack above them is stored in
        r = (TensorSpec((q, w, e), _row_dtype(a.dtype)), TensorSpec((q, w), torch.int32))
        if x.out is not None:
            oa, ob = get_dim_pair(h, x.out)
            assert r[0] == oa, "The dimensions coming from the input and the dimensions of the first output have to match."
            assert r[1] == ob, "The dimensions coming from the input and the dimensions of the second output have to match."
    elif isinstance(x, Pair):
        r = (get_dim_pair(h, x.a), get_dim_pair(h, x.b))
    elif isinstance(x, Zip):
        a, b = get_dim(h, x.a), get_dim(h, x.b)
        assert a == b, "The dimensions of the two inputs to the Zip node have to be equal."
        r = a
    elif isinstance(x, BlockMap):
        r = get_dim(h, x.a)
        assert r.dim[0] == blocks_per_grid(), q_msg % "map"
        check_out(r, x.out)
    elif isinstance(x, BlockRowMap):
        r = get_dim(h, x.a)
        assert r.dim[0] == blocks_per_grid(), q_msg % "row map"
        check_out(r, x.out)
    elif isinstance(x, BlockRowReduce):
        a = get_dim(h, x.a)
        q, w, _ = a.dim
        assert q == blocks_per_grid(), q_msg % "row reduce"
        r = TensorSpec((q, w), _REDUCE_DTYPE[x.f] or a.dtype)
        check_out(r, x.out)
    elif isinstance(x, BlockMatmul):
        a = get_dim(h, x.a)
        q, m, k = a.dim
        assert q == blocks_per_grid(), q_msg % "matmul"
        n, k2 = get_dim(h, x.b).dim
        assert k == k2, "The inner dimensions of the matrix multiplication node have to be equal."
        r = TensorSpec((q, m, n), a.dtype)
    elif isinstance(x, Layer):
        r = x.spec
    elif isinstance(x, KeyGraph):
        r = get_dim_pair(h, x.x)
    elif isinstance(x, Apply):
        a = get_dim(h, x.a)
        r = TensorSpec(a.dim[1:], a.dtype)
    elif isinstance(x, Fst):
        r = get_dim_pair(h, x.x)[0]
    elif isinstance(x, Snd):
        r = get_dim_pair(h, x.x)[1]
    else:
        raise TypeError("Cannot get the dimension of %r." % (x,))
    h[x] = r
    return r


def get_dim(h, x):
    r = get_dim_pair(h, x)
    if not isinstance(r, TensorSpec):
        raise TypeError("The node holds a pair of tensors, not one tensor.")
    return r


def _align(s):
    """`partitionm.align` (corebase/partitionm.spi:3-4)."""
    return (s + 15) // 16 * 16


class Offsets:
    """Where one tensor lives in its arena: `partitionm.offsets` (corebase/partitionm.spi:13-16)."""
    __slots__ = ("spec", "offset")

    def __init__(self, spec, offset):
        self.spec, self.offset = spec, offset


def pass_calculate_partitions(x, dims):
    """Byte offsets of every layer and node output (ml/layers.spi:127-179): depth-first, inputs before the
    node's own output, each tensor aligned to 16 bytes (corebase/partitionm.spi:53-67); node outputs without an
    explicit `out` graph go to the workspace.  Returns [{partition: {node: offsets}, size}] per arena."""
    h_data = [dict() for _ in range(num_spaces())]
    ends = [0] * num_spaces()
    seen = set()

    def place(sid, spec):
        if isinstance(spec, TensorSpec):
            start = _align(ends[sid])
            ends[sid] = start + spec.nbytes
            return Offsets(spec, start)
        return tuple(place(sid, s) for s in spec)

    def g(k, out):
        if out is not None:
            f(out)
        else:
            h_data[workspace_id()][k] = place(workspace_id(), get_dim_pair(dims, k))

    def f(k):
        if k in seen:
            return
        seen.add(k)
        if isinstance(k, (BlockMap, BlockRowMap, BlockRowReduce, BlockRowMapReduce)):
            f(k.a)
            g(k, k.out)
        elif isinstance(k, BlockMatmul):
            f(k.a)
            f(k.b)
            g(k, None)
        elif isinstance(k, (Pair, Zip, Apply)):
            f(k.a)
            f(k.b)
        elif isinstance(k, (Fst, Snd, KeyGraph)):
            f(k.x)
        elif isinstance(k, Layer):
            h_data[k.space_id][k] = place(k.space_id, k.spec)
        elif isinstance(k, KeyScalar):
            pass
        else:
            raise TypeError("unknown graph node %r" % (k,))

    f(x)
    return [{"partition": h, "size": e} for h, e in zip(h_data, ends)]


def create_graph_data(partitions, device="cuda"):
    """One uint8 array per arena (ml/layers.spi:173-179)."""
    return [dict(p, array=torch.empty(p["size"], dtype=torch.uint8, device=device)) for p in partitions]


class Model:
    """`nominal model t = {graph; dims; data}` (ml/layers.spi:60-65)."""

    def __init__(self, graph, dims, data):
        self.graph, self.dims, self.data = graph, dims, data


def create_model(graph, device="cuda"):
    """ml/layers.spi:486-490."""
    dims = {}
    return Model(graph, dims, create_graph_data(pass_calculate_partitions(graph, dims), device))


def model_to_model_ptrs(model):
    """The three arenas, weights / workspace / weight adjoints (ml/layers.spi:495)."""
    return tuple(x["array"] for x in model.data)


def model_ptrs_to_model(graph, ptrs):
    """Rebuild a model around arenas laid out elsewhere (ml/layers.spi:496-502)."""
    dims = {}
    parts = pass_calculate_partitions(graph, dims)
    for p, a in zip(parts, ptrs):
        assert a.dtype == torch.uint8 and a.numel() >= p["size"], \
            "The length of the partition has to be less than or equal to the length of the base array."
    return Model(graph, dims, [dict(p, array=a) for p, a in zip(parts, ptrs)])


def _from_offsets(array, o):
    """`partitionm.from_partition_offsets` (corebase/partitionm.spi:96-105)."""
    if isinstance(o, Offsets):
        return array[o.offset:o.offset + o.spec.nbytes].view(o.spec.dtype).view(o.spec.dim)
    return tuple(_from_offsets(array, x) for x in o)


class LayerState:
    """`nominal layer_state = {rng}` (ml/layers.spi:19-22).  The reference seeds one Philox generator per
    thread for a whole graph run (:339-344); `draws` counts what each of them has handed out so far."""

    def __init__(self, seed=_prim.CONSTANT_SEED):
        self.seed, self.draws = seed, 0

    def rng(self, q, w, cols):
        cfg = _prim.philox(_lib.PHILOX_LAYER, seed=self.seed, threads_per_block=THREADS_PER_BLOCK, blocks_per_grid=q,
                           rows_per_block=w, offset=self.draws)
        rows_per_iteration = THREADS_PER_BLOCK // (cols // 4)
        self.draws += 4 * ((w + rows_per_iteration - 1) // rows_per_iteration)
        return cfg


_MAPS = ("tanh", "sigmoid", "relu", "copy")
_ROW_MAPS = ("ln_l2", "softmax", "regret_matching", "masked_softmax", "masked_regret_matching", "identity")
_ROW_MAP_REDUCES = {"softmax_and_discrete_sample": _lib.ROW_SOFTMAX,
                    "masked_softmax_and_discrete_sample": _lib.ROW_MASKED_SOFTMAX,
                    "regret_matching_and_discrete_sample": _lib.ROW_REGRET_MATCHING,
                    "masked_regret_matching_and_discrete_sample": _lib.ROW_MASKED_REGRET_MATCHING}


def _flat(t):
    return t.reshape(-1, t.shape[-1])


def graph_extract_(layer_state, model, indices):
    """ml/layers.spi:181-252.  With a layer state the nodes are computed on the way; without one the
    tensors are only looked up."""
    data = model.data
    # The tensors of a node are views of the arenas: they are built once per model and arena set (building them on
    # every run cost more host time than the kernels of a small graph take).
    arenas = tuple(x["array"] for x in data)
    cached = model.__dict__.get("_node_views")
    if cached is None or len(cached[0]) != len(arenas) or any(a is not b for a, b in zip(cached[0], arenas)):
        cached = model.__dict__["_node_views"] = (arenas, {})
    views = cached[1]

    def extract_current(node):
        v = views.get(node)
        if v is not None:
            return v
        for x in data:
            if node in x["partition"]:
                v = views[node] = _from_offsets(x["array"], x["partition"][node])
                return v
        raise KeyError("Cannot find the offset in the dictionaries for node %r." % (node,))

    def try_out(node):
        return loop(node.out) if node.out is not None else extract_current(node)

    def loop(graph):
        if isinstance(graph, BlockMap):
            out = try_out(graph)
            if layer_state is not None:
                inner = graph.a
                if graph.f == "relu" and isinstance(inner, BlockMatmul) and out.dtype == extract_current(inner).dtype:
                    # relu of a product: the GEMM's epilogue applies it and writes the map's tensor directly (one
                    # launch and one pass over the activations less; the product's own tensor is not written)
                    a, b = loop(inner.a), loop(inner.b)
                    _matmul.matmul_abt(_flat(a), b, c=_flat(out), alpha=1.0, beta=0.0, relu=True)
                else:
                    _prim.map(graph.f, loop(inner), out)
            return out
        if isinstance(graph, BlockRowMap):
            out = try_out(graph)
            if layer_state is not None:
                a = loop(graph.a)
                _prim._row_map(_prim._ROW_OPS[graph.f], _flat(a), _flat(out), graph.size)
            return out
        if isinstance(graph, BlockRowReduce):
            out = try_out(graph)
            if layer_state is not None:
                a = loop(graph.a)
                if graph.f == "argmax":
                    _prim.row_ops(_flat(a), want=("argmax",), into={"argmax": out.reshape(-1)})
                elif graph.f == "max":
                    _prim.row_ops(_flat(a), want=("rowmax",), into={"rowmax": out.reshape(-1)})
                elif graph.f == "binarize":
                    _prim.binarize(_flat(a), graph.arg, out=out.reshape(-1))
                else:   # discrete_sample
                    q, w, cols = a.shape
                    _prim._sample(_lib.ROW_IDENTITY, _flat(a), rng=layer_state.rng(q, w, cols), want_probs=False,
                                  sample_out=out.reshape(-1))
            return out
        if isinstance(graph, BlockRowMapReduce):
            out_map, out_reduce = try_out(graph)
            if layer_state is not None:
                a = loop(graph.a)
                q, w, cols = a.shape
                _prim._sample(_ROW_MAP_REDUCES[graph.f], _flat(a), rng=layer_state.rng(q, w, cols),
                              mask_size=graph.size, probs_out=_flat(out_map), sample_out=out_reduce.reshape(-1))
            return out_map, out_reduce
        if isinstance(graph, BlockMatmul):
            a, b, out = loop(graph.a), loop(graph.b), extract_current(graph)
            if layer_state is not None:
                # matmul_tf32' false true 1 a b 0 out (ml/layers.spi:227-240)
                _matmul.matmul_abt(_flat(a), b, c=_flat(out), alpha=1.0, beta=0.0)
            return out
        if isinstance(graph, (Zip, Pair)):
            return loop(graph.a), loop(graph.b)
        if isinstance(graph, Fst):
            return loop(graph.x)[0]
        if isinstance(graph, Snd):
            return loop(graph.x)[1]
        if isinstance(graph, Layer):
            return extract_current(graph)
        if isinstance(graph, Apply):
            return loop(graph.a)[loop(graph.b)]
        if isinstance(graph, KeyGraph):
            return loop(graph.x)
        if isinstance(graph, KeyScalar):
            if graph.key not in indices:
                raise KeyError("Cannot extract the node for the graph due to the missing (scalar) key in the "
                               "environment.")
            return indices[graph.key]
        raise TypeError("unknown graph node %r" % (graph,))

    return loop(model.graph)


def graph_extract(model, indices=None):
    """Extracts the tensor at the top level node (ml/layers.spi:255)."""
    return graph_extract_(None, model, indices or {})


def graph_run(model, ls, indices):
    """ml/layers.spi:260."""
    return graph_extract_(ls, model, indices)


def extract_layers_(model, space_id=-1, key=None):
    """All `Layer` nodes of one arena (-1: of all), or the graphs under `key_graph key`, as tensors, in
    graph order (ml/layers.spi:268-307)."""
    found, seen = [], set()

    def f(k):
        if k in seen:
            return
        seen.add(k)
        if isinstance(k, (BlockMap, BlockRowMap, BlockRowReduce, BlockRowMapReduce)):
            f(k.a)
            if k.out is not None:
                f(k.out)
        elif isinstance(k, (BlockMatmul, Apply, Pair, Zip)):
            f(k.a)
            f(k.b)
        elif isinstance(k, (Fst, Snd)):
            f(k.x)
        elif isinstance(k, Layer):
            if key is None and (space_id == -1 or space_id == k.space_id):
                found.append((k.space_id, graph_extract(Model(k, model.dims, model.data)), k.init))
        elif isinstance(k, KeyGraph):
            if key is not None and k.key == key:
                found.append(graph_extract(Model(k.x, model.dims, model.data)))
            else:
                f(k.x)

    f(model.graph)
    return found


def extract_layers(model):
    return extract_layers_(model, -1)


def pass_init(model):
    """Initializes the layers on the host (ml/layers.spi:313)."""
    for _, t, init in extract_layers(model):
        if init is not None:
            init(t)


def _format(t, limit=100):
    if isinstance(t, tuple):
        return ", ".join(_format(x, limit) for x in t)
    return _console.format_tensor(limit, t.detach().cpu().numpy())


def print_layers(model, write=print):
    for _, t, _ in extract_layers(model):
        write(_format(t))


def print_weights(model, write=print):
    for _, t, _ in extract_layers_(model, weight_id()):
        write(_format(t))


def key_extract_list(model, key):
    return extract_layers_(model, key=key)


def key_extract(model, key):
    """The tensor under `key_graph key` (ml/layers.spi:325-330)."""
    found = key_extract_list(model, key)
    if not found:
        raise KeyError("Cannot find the input tensor with the given key.")
    if len(found) > 1:
        raise KeyError("More than one tensor with the given key found.")
    return found[0]


def create_layer_state(seed=_prim.CONSTANT_SEED):
    return LayerState(seed)


def graph_run_device(model, ls, indices):
    graph_run(model, ls, indices)


def _build_fused_run(model, plan, ls, static_weights=False):
    """The closure graph_run_host calls for a graph that sp_mlp_forward can run: every argument is prepared here.
    static_weights: the caller vouches that the weights stay as they are now; they are then packed once, here, and the
    runs go to the packed kernel (sp_mlp_forward_packed) when it takes the stack."""
    x_node, w_nodes, top, head = plan
    x = _flat(graph_extract(Model(x_node, model.dims, model.data)))
    ws = [graph_extract(Model(w, model.dims, model.data)) for w in w_nodes]
    probs, action = graph_extract(model)
    q, w, cols = probs.shape
    rng = ls.rng(q, w, cols)
    policy, act = _flat(probs), action.reshape(-1)
    n = len(ws)
    dims = [x.shape[1]] + [t.shape[0] for t in ws]
    for i, t in enumerate(ws):
        if t.dtype != x.dtype:
            raise TypeError("weights[%d] must have the dtype of x" % i)
        assert t.shape[1] == dims[i], "The K dimension of the A and B tensors must match."
    wp = (C.c_void_p * n)(*[ptr(t, name="weights[%d]" % i) for i, t in enumerate(ws)])
    dp = (C.c_int32 * (n + 1))(*dims)
    # The head draws its uniforms inside the kernel, from the stream a run of the reference starts at its seed
    # (ml/layers.spi:339-344): no uniform tensor, no launch of its own, nothing carried over from run to run.
    args = (_lib.DTYPES[x.dtype], ptr(x, name="x"), n, wp, None, dp, None, C.byref(rng),
            ptr(policy, torch.float32, "policy_out"), ptr(act, torch.int32, "action_out"), None, x.shape[0], HEADS[head],
            top.size)
    keep = (x, ws, probs, action, rng, policy, act)   # the views stay alive as long as the closure does

    packed = pack_weights(ws) if static_weights else None
    if packed is not None and builtins.min(dims[-1], top.size or dims[-1]) <= 16:
        pargs = args[:3] + (ptr(packed.buffer), packed.buffer.numel()) + args[4:]
        keep = keep + (packed,)

        def run_packed():
            check(lib.sp_mlp_forward_packed(*pargs, stream_ptr()))
            return keep

        return run_packed

    def run():
        check(lib.sp_mlp_forward(*args, stream_ptr()))
        return keep

    return run


def _fused_plan(model):
    """A `matmul -> relu -> ... -> matmul -> head` chain over 16-bit tensors that sp_mlp_forward can run:
    returns (input node, [weight nodes], head node) or None."""
    top = model.graph
    head_ops = {"softmax_and_discrete_sample": "softmax", "masked_softmax_and_discrete_sample": "softmax",
                "regret_matching_and_discrete_sample": "regret_matching",
                "masked_regret_matching_and_discrete_sample": "regret_matching"}
    if not isinstance(top, BlockRowMapReduce) or top.f not in head_ops:
        return None
    weights, node = [], top.a
    while True:
        if not isinstance(node, BlockMatmul) or not isinstance(node.b, Layer):
            return None
        weights.append(node.b)
        node = node.a
        if isinstance(node, BlockMap) and node.f == "relu" and node.out is None:
            node = node.a
            continue
        break
    while isinstance(node, KeyGraph):
        node = node.x
    if not isinstance(node, Layer):
        return None
    weights.reverse()
    dims = [node.spec.dim[-1]] + [w.spec.dim[0] for w in weights]
    ok = node.spec.dtype in (torch.float16, torch.bfloat16) and all(w.spec.dtype == node.spec.dtype for w in weights)
    # the shapes sp_mlp_forward takes (`max` is a node constructor in this module, hence builtins.max)
    ok = ok and builtins.max(dims) <= 256 and dims[0] % 16 == 0 and all(d % 32 == 0 for d in dims[1:-1]) and dims[-1] <= 64
    return (node, weights, top, head_ops[top.f]) if ok else None


def _sampling_draws(w, cols):
    """32-bit draws one sampling node takes from every thread's generator: 4 per row-iteration."""
    rows_per_iteration = THREADS_PER_BLOCK // (cols // 4)
    return 4 * ((w + rows_per_iteration - 1) // rows_per_iteration)


def _batchable_key(model, sizes):
    """The key of `sizes` if the whole loop over it can run as one batched pass: a single key that the
    graph only uses to index leading dimensions (`apply key tensor`)."""
    if len(sizes) != 1:
        return None
    (key,) = sizes
    ok = [True]

    def f(k, under_apply=False):
        if isinstance(k, KeyScalar):
            ok[0] = ok[0] and under_apply and k.key == key
        elif isinstance(k, (BlockMap, BlockRowMap, BlockRowReduce, BlockRowMapReduce)):
            f(k.a)
            if k.out is not None:
                f(k.out)
        elif isinstance(k, Apply):
            f(k.a)
            f(k.b, True)
        elif isinstance(k, (BlockMatmul, Pair, Zip)):
            f(k.a)
            f(k.b)
        elif isinstance(k, (Fst, Snd, KeyGraph)):
            f(k.x)

    f(model.graph)
    return key if ok[0] else None


_ENSEMBLE_HEADS = {"softmax": "softmax", "masked_softmax": "softmax", "regret_matching": "regret_matching",
                   "masked_regret_matching": "regret_matching", "softmax_and_discrete_sample": "softmax",
                   "masked_softmax_and_discrete_sample": "softmax",
                   "regret_matching_and_discrete_sample": "regret_matching",
                   "masked_regret_matching_and_discrete_sample": "regret_matching"}


def _fused_ensemble_plan(model, key):
    """`input -> matmul_ensemble [-> relu -> matmul_ensemble] -> head` over f32 tensors with the members' outputs stacked
    under `apply key` -- the graphs of the reference's agents (game/leduc/model_cem.spi:55-63,
    game/nl_hu_holdem/model_cem.spi:84-100: a policy head; game/leduc/model_cfr.spi:56-61,
    game/nl_hu_holdem/model_cfr.spi:82-88: one layer and `binarize'`):
    (x node, [stacked weight nodes], stacked output node(s), top node) or None."""
    top = model.graph

    def passive(k):   # tensors only, nothing to compute: the tables a model keeps beside its network
        if isinstance(k, (Layer, KeyScalar)):
            return True
        if isinstance(k, (KeyGraph, Fst, Snd)):
            return passive(k.x)
        if isinstance(k, (Pair, Zip, Apply)):
            return passive(k.a) and passive(k.b)
        return False

    while isinstance(top, Pair) and passive(top.b):
        top = top.a
    sampling = isinstance(top, BlockRowMapReduce)
    hashing = isinstance(top, BlockRowReduce) and top.f == "binarize"
    if not hashing and (not isinstance(top, (BlockRowMap, BlockRowMapReduce)) or top.f not in _ENSEMBLE_HEADS):
        return None
    if top.out is None:
        return None

    def stacked(k):   # `apply key t` -> t
        while isinstance(k, KeyGraph):
            k = k.x
        if isinstance(k, Apply) and isinstance(k.b, KeyScalar) and k.b.key == key and passive(k.a):
            return k.a
        return None

    if sampling:
        out = top.out
        while isinstance(out, KeyGraph):
            out = out.x
        if not isinstance(out, Pair):
            return None
        outs = (stacked(out.a), stacked(out.b))
    else:
        outs = (stacked(top.out),)
    if any(o is None for o in outs):
        return None
    last = top.a
    if not isinstance(last, BlockMatmul):
        return None
    weights = [stacked(last.b)]
    x = last.a
    if isinstance(x, BlockMap):
        if hashing or not (x.f == "relu" and x.out is None and isinstance(x.a, BlockMatmul)):
            return None
        weights.insert(0, stacked(x.a.b))
        x = x.a.a
    while isinstance(x, KeyGraph):
        x = x.x
    if any(w is None for w in weights) or not isinstance(x, Layer):
        return None
    return x, weights, outs, top


def _run_fused_ensemble(model, key, count, ls):
    """One sp_mlp_forward_ensemble / sp_ensemble_binarize launch in place of the batched pass, where the graph is of
    that shape."""
    plan = _fused_ensemble_plan(model, key)
    if plan is None:
        return False
    x_node, w_nodes, out_nodes, top = plan
    tensor = lambda node: graph_extract(Model(node, model.dims, model.data))
    x, ws = tensor(x_node), [tensor(w) for w in w_nodes]
    first_out = tensor(out_nodes[0])
    if x.dim() != 3 or any(w.dim() != 3 or w.dtype != torch.float32 or w.shape[0] != count for w in ws) or x.dtype != torch.float32:
        return False
    q, w, k0 = x.shape
    cols = ws[-1].shape[1]
    if ws[0].shape[2] != k0 or k0 % 8 != 0 or k0 < 8:
        return False
    if isinstance(top, BlockRowReduce):           # binarize
        if len(ws) != 1 or k0 > 256 or first_out.shape != (count, q, w) or first_out.dtype != torch.int32 or top.arg <= 0:
            return False
        ensemble_binarize(_flat(x), ws[0], top.arg, first_out.reshape(count, q * w))
        return True
    probs = first_out
    computed = top.size or cols
    if len(ws) == 2 and not (ws[0].shape[1] == ws[1].shape[2] == 64 and k0 <= 128):
        return False
    if not (k0 <= 256 and cols <= 64 and computed <= 4 and probs.dtype == torch.float32 and probs.shape == (count, q, w, cols)):
        return False
    action, rng = None, None
    if len(out_nodes) == 2:
        action = tensor(out_nodes[1])
        if action.shape != (count, q, w) or action.dtype != torch.int32 or cols % 4 != 0:
            return False
        # member e draws what the e-th sequential run would: every run takes one sampling node's draws
        draws = _sampling_draws(w, cols)
        rng = _prim.philox(_lib.PHILOX_LAYER, seed=ls.seed, threads_per_block=THREADS_PER_BLOCK, blocks_per_grid=q,
                           rows_per_block=w, offset=ls.draws, member_rows=q * w, member_draws=draws)
        ls.draws += draws
    mlp_forward_ensemble(_flat(x), ws, _ENSEMBLE_HEADS[top.f], None, top.size, probs.reshape(count, q * w, cols),
                         action.reshape(count, q * w) if action is not None else None, rng)
    return True


def _graph_run_batched(model, key, count, ls):
    """`loop.linear {key=count} fun indices => graph_run_device m ls indices` (ml/layers.spi:343-344) as ONE
    pass: `apply key t` yields the whole tensor, every node downstream works on `count` stacked members
    (temporaries outside the workspace arena, which is sized for one member), matmuls become one
    strided-batched launch, and sampling nodes draw for member e what the e-th sequential run would."""
    data, dims = model.data, model.dims
    tmp = model.__dict__.setdefault("_batched_tmp", {})

    def count_draws(k):
        if isinstance(k, (BlockRowReduce, BlockRowMapReduce)):
            sampling = isinstance(k, BlockRowMapReduce) or k.f == "discrete_sample"
            _, w, cols = get_dim(dims, k.a).dim
            return count_draws(k.a) + (_sampling_draws(w, cols) if sampling else 0)
        if isinstance(k, (BlockMap, BlockRowMap)):
            return count_draws(k.a)
        if isinstance(k, (BlockMatmul, Pair, Zip)):
            return count_draws(k.a) + count_draws(k.b)
        if isinstance(k, (Fst, Snd, KeyGraph)):
            return count_draws(k.x)
        if isinstance(k, Apply):
            return count_draws(k.a)
        return 0

    draws_per_run = count_draws(model.graph)

    def extract_current(node):
        for x in data:
            if node in x["partition"]:
                return _from_offsets(x["array"], x["partition"][node])
        raise KeyError("Cannot find the offset in the dictionaries for node %r." % (node,))

    def stacked(t, spec):
        return t.dim() == len(spec.dim) + 1

    def out_for(node, batched):
        if getattr(node, "out", None) is not None:
            return loop(node.out)
        if not batched:
            return extract_current(node)
        if node not in tmp:
            spec = get_dim_pair(dims, node)
            device = data[workspace_id()]["array"].device
            make = lambda sp: torch.empty((count,) + sp.dim, dtype=sp.dtype, device=device)
            tmp[node] = make(spec) if isinstance(spec, TensorSpec) else tuple(make(sp) for sp in spec)
        return tmp[node]

    def rng(a, batched):
        q, w, cols = a.shape[-3:]
        cfg = _prim.philox(_lib.PHILOX_LAYER, seed=ls.seed, threads_per_block=THREADS_PER_BLOCK, blocks_per_grid=q,
                           rows_per_block=w, offset=ls.draws, member_rows=q * w if batched else 0,
                           member_draws=draws_per_run)
        ls.draws += _sampling_draws(w, cols)
        return cfg

    def loop(graph):
        if isinstance(graph, BlockMap):
            a = loop(graph.a)
            out = out_for(graph, stacked(a, get_dim(dims, graph.a)))
            assert out.shape == a.shape, "a batched input needs a batched output tensor"
            _prim.map(graph.f, a, out)
            return out
        if isinstance(graph, BlockRowMap):
            a = loop(graph.a)
            out = out_for(graph, stacked(a, get_dim(dims, graph.a)))
            assert out.shape == a.shape, "a batched input needs a batched output tensor"
            _prim._row_map(_prim._ROW_OPS[graph.f], _flat(a), _flat(out), graph.size)
            return out
        if isinstance(graph, BlockRowReduce):
            a = loop(graph.a)
            batched = stacked(a, get_dim(dims, graph.a))
            out = out_for(graph, batched)
            assert out.shape == a.shape[:-1], "a batched input needs a batched output tensor"
            if graph.f == "argmax":
                _prim.row_ops(_flat(a), want=("argmax",), into={"argmax": out.reshape(-1)})
            elif graph.f == "max":
                _prim.row_ops(_flat(a), want=("rowmax",), into={"rowmax": out.reshape(-1)})
            elif graph.f == "binarize":
                _prim.binarize(_flat(a), graph.arg, out=out.reshape(-1))
            else:
                _prim._sample(_lib.ROW_IDENTITY, _flat(a), rng=rng(a, batched), want_probs=False,
                              sample_out=out.reshape(-1))
            return out
        if isinstance(graph, BlockRowMapReduce):
            a = loop(graph.a)
            batched = stacked(a, get_dim(dims, graph.a))
            out_map, out_reduce = out_for(graph, batched)
            assert out_map.shape == a.shape, "a batched input needs batched output tensors"
            _prim._sample(_ROW_MAP_REDUCES[graph.f], _flat(a), rng=rng(a, batched), mask_size=graph.size,
                          probs_out=_flat(out_map), sample_out=out_reduce.reshape(-1))
            return out_map, out_reduce
        if isinstance(graph, BlockMatmul):
            a, b = loop(graph.a), loop(graph.b)
            ab, bb = stacked(a, get_dim(dims, graph.a)), stacked(b, get_dim(dims, graph.b))
            out = out_for(graph, ab or bb)
            if not (ab or bb):
                _matmul.matmul_abt(_flat(a), b, c=_flat(out), alpha=1.0, beta=0.0)
            else:
                a3 = a.reshape(count, -1, a.shape[-1]) if ab else _flat(a)
                _matmul.matmul_abt_batched(a3, b, c=out.reshape(count, -1, out.shape[-1]), alpha=1.0, beta=0.0)
            return out
        if isinstance(graph, (Zip, Pair)):
            return loop(graph.a), loop(graph.b)
        if isinstance(graph, Fst):
            return loop(graph.x)[0]
        if isinstance(graph, Snd):
            return loop(graph.x)[1]
        if isinstance(graph, Layer):
            return extract_current(graph)
        if isinstance(graph, Apply):
            t = loop(graph.a)
            assert t.shape[0] == count, "the key's size must be the tensor's leading dimension"
            return t          # the key is the batch: all members at once
        if isinstance(graph, KeyGraph):
            return loop(graph.x)
        raise TypeError("unknown graph node %r" % (graph,))

    return loop(model.graph)


def weights_changed(model):
    """Forget what was prepared from the current weights (the packed copy behind `static_weights=True`): call it
    after writing new values into the weights arena."""
    model.__dict__.pop("_fused_runs", None)


def graph_run_host(model, sizes=None, seed=_prim.CONSTANT_SEED, fuse=True, batched=True, static_weights=False):
    """Runs the graph for every combination of the key indices in `sizes`, e.g. {"ensemble": 16}
    (ml/layers.spi:336-344).  Uniforms come from the reference's per-thread Philox streams.  A loop over
    one key that only indexes leading dimensions runs as a single batched pass with the same results
    (`batched=False` keeps the member-by-member loop).  `static_weights=True` says that the weights have not
    changed since the previous such run (or since `weights_changed(model)`): a fused relu-MLP then keeps a copy
    of them packed for the faster kernel instead of reading the arena on every run."""
    if fuse and not sizes:
        # The plan of a model does not change between runs: the tensors are views of its arenas and the
        # generator restarts with every run.  It is built once per (model, seed); a call then costs one
        # C-ABI call instead of a walk over the graph (which took several times as long as the kernel).
        cache = model.__dict__.get("_fused_runs")
        if cache is None:
            cache = model.__dict__["_fused_runs"] = {}
        entry = cache.get((seed, static_weights))
        if entry is not None:
            arenas, run = entry
            data = model.data
            if arenas[0] is data[0]["array"] and arenas[1] is data[1]["array"] and arenas[2] is data[2]["array"]:
                if run:
                    run()
                    return
            else:
                entry = None    # the model was given other arenas: plan again
        if entry is None:
            plan = _fused_plan(model)
            run = _build_fused_run(model, plan, create_layer_state(seed), static_weights) if plan is not None else False
            cache[(seed, static_weights)] = (tuple(d["array"] for d in model.data), run)
            if run:
                run()
                return
    sizes = sizes or {}
    # What a run launches depends on the graph, the arenas, the key sizes and the seed only (every sampling node draws
    # from a generator that restarts with the run), so the first run is recorded and later runs replay its launches;
    # walking the graph took longer than the kernels of a small graph.
    tapes = model.__dict__.get("_tapes")
    if tapes is None:
        tapes = model.__dict__["_tapes"] = {}
    tape_key = (seed, fuse, batched, tuple(sorted(sizes.items())))
    entry = tapes.get(tape_key)
    data = model.data
    if entry is not None and len(entry[0]) == len(data) and all(a is d["array"] for a, d in zip(entry[0], data)):
        entry[1].replay()
        return
    tape = _lib.start_tape()
    try:
        _graph_run_walk(model, sizes, seed, batched, fuse)
    finally:
        _lib.stop_tape()
    tapes[tape_key] = (tuple(d["array"] for d in data), tape)


def _graph_run_walk(model, sizes, seed, batched, fuse=True):
    """One run by walking the graph: a single batched pass over one key where that is possible (a single fused launch
    where the graph is a two-layer relu stack per member), else every combination of the key indices in turn."""
    ls = create_layer_state(seed)
    key = _batchable_key(model, sizes) if batched and sizes else None
    if key is not None and sizes[key] > 1:
        if not (fuse and _run_fused_ensemble(model, key, sizes[key], ls)):
            _graph_run_batched(model, key, sizes[key], ls)
        return
    keys = list(sizes)
    for combo in itertools.product(*[range(sizes[k]) for k in keys]):
        graph_run_device(model, ls, dict(zip(keys, combo)))


# ---- node constructors (ml/layers.spi:346-484) ------------------------------------------------

def _curried(f):
    """f(args..., x) -> also callable without x, giving the function of x (for `pipe`)."""
    def g(*args):
        if args and isinstance(args[-1], Graph):
            return f(*args)
        return lambda x: f(*(args + (x,)))
    g.__name__, g.__doc__ = f.__name__, f.__doc__
    return g


def pipe(x, *fs):
    """x |> f1 |> f2 ..."""
    for f in fs:
        x = f(x)
    return x


def tanh(x):
    return BlockMap("tanh", x)


def sigmoid(x):
    return BlockMap("sigmoid", x)


def relu(x):
    """relu = max 0 (ml/layers.spi:355)."""
    return BlockMap("relu", x)


@_curried
def max_(out, x):
    return BlockRowReduce("max", x, out)


def max(x):  # noqa: A001  (the reference's name, ml/layers.spi:361)
    return BlockRowReduce("max", x)


def ln_l2(x):
    return BlockRowMap("ln_l2", x)


def argmax(x):
    return BlockRowReduce("argmax", x)


@_curried
def softmax_(out, x):
    return BlockRowMap("softmax", x, out)


def softmax(x):
    return BlockRowMap("softmax", x)


@_curried
def regret_matching_(out, x):
    return BlockRowMap("regret_matching", x, out)


def regret_matching(x):
    return BlockRowMap("regret_matching", x)


@_curried
def discrete_sample_(out, x):
    return BlockRowReduce("discrete_sample", x, out)


def discrete_sample(x):
    return BlockRowReduce("discrete_sample", x)


@_curried
def softmax_and_discrete_sample_(out, x):
    return BlockRowMapReduce("softmax_and_discrete_sample", x, out)


def softmax_and_discrete_sample(x):
    return BlockRowMapReduce("softmax_and_discrete_sample", x)


@_curried
def copy_(out, x):
    return BlockMap("copy", x, out)


def copy(x):
    return BlockMap("copy", x)


@_curried
def masked_softmax_(size, out, x):
    return BlockRowMap("masked_softmax", x, out, size)


@_curried
def masked_softmax(size, x):
    return BlockRowMap("masked_softmax", x, None, size)


@_curried
def masked_regret_matching_(size, out, x):
    return BlockRowMap("masked_regret_matching", x, out, size)


@_curried
def masked_regret_matching(size, x):
    return BlockRowMap("masked_regret_matching", x, None, size)


@_curried
def masked_softmax_and_discrete_sample_(size, out, x):
    return BlockRowMapReduce("masked_softmax_and_discrete_sample", x, out, size)


@_curried
def masked_softmax_and_discrete_sample(size, x):
    return BlockRowMapReduce("masked_softmax_and_discrete_sample", x, None, size)


@_curried
def binarize_(modulo, out, x):
    return BlockRowReduce("binarize", x, out, modulo)


@_curried
def binarize(modulo, x):
    return BlockRowReduce("binarize", x, None, modulo)


def key_scalar(key):
    return KeyScalar(key)


def key_graph(key, x):
    return KeyGraph(key, x)


def apply(b, a):  # noqa: A001  (the reference's name, ml/layers.spi:450)
    """Index the leading dimension of `a` with the run-time value of key `b`."""
    return Apply(a, key_scalar(b))


def pair(a, b):
    return Pair(a, b)


def fst_(x):
    return Fst(x)


def snd_(x):
    return Snd(x)


def layer(space_id, dim, init=None, dtype="float"):
    return Layer(space_id, dim, init, dtype)


tensor = layer


def init_const(t, v):
    t.fill_(v)


def init_zero(t):
    t.zero_()


def weight_init(t, std=0.1):
    """`weight_init` (ml/layers.spi:460-463): N(0, 0.1) in the current source."""
    t.copy_(torch.randn(t.shape, generator=_gen(t.device), device=t.device, dtype=torch.float32) * std)


def weight_(dim, init, dtype="float"):
    return Layer(weight_id(), dim, init, dtype)


def weight(dim, dtype="float"):
    return weight_(dim, weight_init, dtype)


@_curried
def matmul(ba, x):
    """`matmul (in, out) x = BlockMatmul(x, weight (out, in))` (ml/layers.spi:467): the weight is stored
    (out_features, in_features) row-major, the B operand of A.B^T."""
    b, a = ba
    return BlockMatmul(x, weight((a, b), _input_dtype(x)))


@_curried
def matmul_ensemble(cba, x):
    """E weight matrices (E, out, in) under the key "weights", indexed by the run-time key "ensemble"
    (ml/layers.spi:468-471)."""
    c, b, a = cba
    weights = key_graph("weights", Layer(weight_id(), (c, a, b), weight_init, _input_dtype(x)))
    return BlockMatmul(x, apply("ensemble", weights))


@_curried
def matmul_ensemble_with_adjoint(cba, x):
    """`matmul_ensemble_with_adjoint (c, b, a) x` (ml/layers.spi:472-479): the E weight matrices (E, out, in) in the
    weights arena under the key "weights" AND their transposed dual ((out, in), E) in the weight-adjoint arena, the
    pair under the key "cem_weight_layer_dual" -- the two tensors the CEM update transposes between
    (`grid_transpose weights transposed_weights`, ml/cem.spi:131-146).  The product reads the first of the pair."""
    c, b, a = cba
    dtype = _input_dtype(x)
    dual = key_graph("cem_weight_layer_dual",
                     pair(key_graph("weights", Layer(weight_id(), (c, a, b), weight_init, dtype)),
                          Layer(weight_adjoint_id(), (a, b, c), None, dtype)))
    return BlockMatmul(x, apply("ensemble", fst_(dual)))


def _input_dtype(x):
    return get_dim({}, x).dtype


def input_(dim, dtype="float"):
    """Creates a layer in the workspace.  Doesn't initialize it (ml/layers.spi:481)."""
    return Layer(workspace_id(), dim, None, dtype)


def input(key, dim, dtype="float"):  # noqa: A001  (the reference's name, ml/layers.spi:482-484)
    return key_graph(key, input_(dim, dtype))


# ----------------------------------------------------------------------------------------------
# the reference's self-tests (ml/layers.spi:510-668), same files, same text format
# ----------------------------------------------------------------------------------------------

def _redirect(root, name):
    import os
    d = os.path.join(root, name)
    os.makedirs(d, exist_ok=True)
    return open(os.path.join(d, "layers.txt"), "w")


def _fill_normal(t):
    t.copy_(torch.randn(t.shape, generator=_gen(t.device), device=t.device, dtype=torch.float32))


def test1(root="test_text_outputs/layers/"):
    """Tests whether randomly initializing the params of the graph works."""
    set_random_seed()
    with _redirect(root, "test1") as f:
        w = lambda s: f.write(s + "\n")
        graph = pipe(input("input", (blocks_per_grid(), 1, 4)), matmul((4, 4)), tanh, matmul((4, 4)), tanh,
                     matmul((4, 2)), tanh)
        model = create_model(graph)
        for x in model.data:
            x["array"].zero_()
        w("---")
        print_weights(model, w)
        pass_init(model)
        w("Done initing.")
        print_weights(model, w)
    return model


def test2(root="test_text_outputs/layers/"):
    """Tests whether extracting the inputs of the graph works.  Also randomly inits them."""
    set_random_seed()
    with _redirect(root, "test2") as f:
        w = lambda s: f.write(s + "\n")
        graph = pipe(input("input", (blocks_per_grid(), 1, 2)), matmul((2, 4)), tanh, matmul((4, 4)), tanh,
                     matmul((4, 2)), tanh)
        model = create_model(graph)
        w("---")
        pass_init(model)
        w("Here are the weight matrices.")
        print_weights(model, w)
        w("Here is the input tensor.")
        x = key_extract(model, "input")
        _fill_normal(x)
        w(_format(x))
    return model


def test3(root="test_text_outputs/layers/"):
    """Tests running a feedforward model which outputs the sampling indices."""
    set_random_seed()
    with _redirect(root, "test3") as f:
        w = lambda s: f.write(s + "\n")
        graph = pipe(input("input", (blocks_per_grid(), 64, 64)), matmul((64, 64)), ln_l2, relu, matmul((64, 64)),
                     ln_l2, relu, matmul((64, 64)), softmax_and_discrete_sample)
        model = create_model(graph)
        pass_init(model)
        w("Here are the weight matrices.")
        print_weights(model, w)
        x = key_extract(model, "input")
        _fill_normal(x)
        w(_format(x))
        w("Here is the output tensor.")
        graph_run_host(model, {})
        w(_format(graph_extract(model, {})))
        w("====")
    return model


def _ensemble_test(name, ensemble, size, deep, root):
    set_random_seed()
    with _redirect(root, name) as f:
        w = lambda s: f.write(s + "\n")
        q = blocks_per_grid()
        out = pair(apply("ensemble", input("output_probs", (ensemble, q, 64, 64))),
                   apply("ensemble", input("output_indices", (ensemble, q, 64), "int")))
        x = pipe(input("input", (q, 64, 64)), matmul_ensemble((ensemble, 64, 64)))
        if deep:
            x = pipe(x, ln_l2, relu, matmul_ensemble((ensemble, 64, 64)), ln_l2, relu,
                     matmul_ensemble((ensemble, 64, 64)))
        graph = softmax_and_discrete_sample_(out, x) if size is None else \
            masked_softmax_and_discrete_sample_(size, out, x)
        model = create_model(graph)
        pass_init(model)
        if deep:
            w("Here are the weight matrices.")
            print_weights(model, w)
        inp = key_extract(model, "input")
        _fill_normal(inp)
        if deep:
            w(_format(inp))
            w("Here is the output tensor.")
        graph_run_host(model, {"ensemble": ensemble})
        w(_format(key_extract(model, "output_indices"), limit=2 ** 31 - 1))
    return model


def test4(root="test_text_outputs/layers/"):
    """Tests running a feedforward ensemble model which keeps around the sampling probabilities."""
    return _ensemble_test("test4", 16, None, True, root)


def test5(root="test_text_outputs/layers/"):
    """... with masking."""
    return _ensemble_test("test5", 4, 11, False, root)


def main_body(root="test_text_outputs/layers/"):
    test1(root)
    test2(root)
    test3(root)
    test4(root)
    test5(root)


def main():
    main_body()
    torch.cuda.synchronize()
    return 0
