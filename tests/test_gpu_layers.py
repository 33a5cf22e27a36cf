"""The layer graph on the GPU (every node through the C ABI) against the NumPy oracle composed by
hand the way ml/layers.spi:194-240 interprets the nodes.  Bar: f32 tensors within a relative
Frobenius error of 1e-5, 16-bit stacks 3e-3; sampled indices bit-exact given the kernel's own
probabilities and the reference's per-thread Philox streams.

PARITY UNPINNED against reference outputs: the reference's layer goldens hold inputs truncated to 100
values, so no forward result can be recomputed from them; what they do pin (arena sizes, text
format) is in test_layers_graph_cpu.py."""
import os

import numpy as np
import pytest
import torch

from oracle import gemm as ogemm, layers as olayers, philox as ophilox, row_ops as orow
from gpu_util import announce, dev, host

pytestmark = pytest.mark.gpu

Q = 24   # blocks per grid of the reference's RTX 4060 runs


@pytest.fixture()
def L():
    from ml import layers
    layers.set_blocks_per_grid(Q)
    layers.set_random_seed(5)
    return layers


def fill(t, rng, scale=1.0):
    x = (rng.standard_normal(tuple(t.shape)) * scale).astype(np.float32)
    t.copy_(torch.from_numpy(x).to(t.dtype))
    return host(t.float()) if t.dtype != torch.float32 else x


def dense_ln_relu(h, ws):
    """matmul -> ln_l2 -> relu -> ... -> matmul on (rows, k) f32."""
    for i, w in enumerate(ws):
        h = ogemm.gemm_abt(h, w)
        if i + 1 < len(ws):
            h = orow.relu(orow.ln_l2(h))
    return h


def test_feedforward_sampling_graph(L):
    """The graph of ml/layers.spi test3 (:564-593)."""
    announce("layers test3 graph")
    g = L.pipe(L.input("input", (Q, 64, 64)), L.matmul((64, 64)), L.ln_l2, L.relu, L.matmul((64, 64)), L.ln_l2, L.relu,
               L.matmul((64, 64)), L.softmax_and_discrete_sample)
    m = L.create_model(g)
    L.pass_init(m)
    rng = np.random.default_rng(0)
    x = fill(L.key_extract(m, "input"), rng)
    ws = [host(t) for _, t, _ in L.extract_layers_(m, L.weight_id())]
    assert [w.shape for w in ws] == [(64, 64)] * 3 and 0.08 < ws[0].std() < 0.12
    L.graph_run_host(m, {})
    probs, idx = (host(t) for t in L.graph_extract(m, {}))
    want = orow.softmax(dense_ln_relu(x.reshape(-1, 64), ws))
    assert ogemm.rel_frobenius(probs.reshape(-1, 64), want) < 1e-5
    u = ophilox.row_uniforms_layer(Q, 64, 64)
    assert (idx.reshape(-1) == orow.discrete_sampling(probs.reshape(-1, 64), u, order="wave")).all()
    # a second run redraws from the start of every thread's stream, like a second kernel launch
    L.graph_run_host(m, {})
    assert (host(L.graph_extract(m, {})[1]) == idx).all()


@pytest.mark.parametrize("ensemble,size,deep", [(3, None, True), (4, 11, False)])
def test_ensemble_graphs(L, ensemble, size, deep):
    """The graphs of ml/layers.spi test4 (:596-630) and test5 (:633-665), smaller ensembles."""
    announce("layers ensemble graph e=%d size=%s" % (ensemble, size))
    out = L.pair(L.apply("ensemble", L.input("output_probs", (ensemble, Q, 64, 64))),
                 L.apply("ensemble", L.input("output_indices", (ensemble, Q, 64), "int")))
    x = L.pipe(L.input("input", (Q, 64, 64)), L.matmul_ensemble((ensemble, 64, 64)))
    if deep:
        x = L.pipe(x, L.ln_l2, L.relu, L.matmul_ensemble((ensemble, 64, 64)), L.ln_l2, L.relu,
                   L.matmul_ensemble((ensemble, 64, 64)))
    g = L.softmax_and_discrete_sample_(out, x) if size is None else L.masked_softmax_and_discrete_sample_(size, out, x)
    m = L.create_model(g)
    L.pass_init(m)
    rng = np.random.default_rng(1)
    xin = fill(L.key_extract(m, "input"), rng)
    ws = [host(t) for t in L.key_extract_list(m, "weights")]
    assert all(w.shape == (ensemble, 64, 64) for w in ws) and len(ws) == (3 if deep else 1)
    L.graph_run_host(m, {"ensemble": ensemble})
    probs, idx = host(L.key_extract(m, "output_probs")), host(L.key_extract(m, "output_indices"))
    per_node = ophilox.draws_per_sampling_node(64, 64)
    for e in range(ensemble):
        logits = dense_ln_relu(xin.reshape(-1, 64), [w[e] for w in ws])
        want = orow.softmax(logits) if size is None else orow.masked_softmax(logits, size)
        assert ogemm.rel_frobenius(probs[e].reshape(-1, 64), want) < 1e-5
        # one generator state per thread for the whole run: ensemble member e starts e nodes in
        u = ophilox.row_uniforms_layer(Q, 64, 64, offset=e * per_node)
        assert (idx[e].reshape(-1) == orow.discrete_sampling(probs[e].reshape(-1, 64), u, order="wave")).all()
        if size is not None:
            assert (idx[e] < size).all() and (probs[e][..., size:] == 0).all()


def test_batched_ensemble_pass_equals_member_by_member_loop(L):
    """`graph_run_host model {ensemble}` as one batched pass (strided-batched GEMMs, stacked row ops, per-member
    Philox offsets) gives bit for bit what the loop over the members gives."""
    announce("layers batched ensemble pass")
    ensemble = 6
    out = L.pair(L.apply("ensemble", L.input("output_probs", (ensemble, Q, 64, 64))),
                 L.apply("ensemble", L.input("output_indices", (ensemble, Q, 64), "int")))
    x = L.pipe(L.input("input", (Q, 64, 64)), L.matmul_ensemble((ensemble, 64, 64)), L.ln_l2, L.relu,
               L.matmul_ensemble((ensemble, 64, 32)), L.tanh, L.matmul((32, 64)))
    g = L.masked_softmax_and_discrete_sample_(17, out, x)
    m = L.create_model(g)
    L.pass_init(m)
    fill(L.key_extract(m, "input"), np.random.default_rng(8))
    assert L._batchable_key(m, {"ensemble": ensemble}) == "ensemble"
    L.graph_run_host(m, {"ensemble": ensemble}, batched=False)
    want_p, want_i = host(L.key_extract(m, "output_probs")).copy(), host(L.key_extract(m, "output_indices")).copy()
    L.key_extract(m, "output_probs").zero_()
    L.key_extract(m, "output_indices").zero_()
    L.graph_run_host(m, {"ensemble": ensemble})
    assert (host(L.key_extract(m, "output_probs")) == want_p).all()
    assert (host(L.key_extract(m, "output_indices")) == want_i).all()
    assert (want_i < 17).all() and len(np.unique(want_i)) > 5


def test_ensemble_with_adjoint_and_the_cem_update(L):
    """`matmul_ensemble_with_adjoint` keeps every ensemble layer as the pair (weights, transposed dual in the adjoint
    arena); the product is the one `matmul_ensemble` computes, and the reference's CEM update walks the pair:
    transpose into the dual, resample the losers there, weight norms, transpose back (ml/cem.spi:120-146)."""
    from ml import primitives as P
    announce("layers ensemble with adjoint + CEM update")
    ensemble = 8
    def graph(ctor):
        out = L.pair(L.apply("ensemble", L.input("output_probs", (ensemble, Q, 16, 64))),
                     L.apply("ensemble", L.input("output_indices", (ensemble, Q, 16), "int")))
        return L.softmax_and_discrete_sample_(out, L.pipe(L.input("input", (Q, 16, 32)), ctor((ensemble, 32, 64))))
    m = L.create_model(graph(L.matmul_ensemble_with_adjoint))
    ref = L.create_model(graph(L.matmul_ensemble))
    sizes = [x["array"].numel() for x in m.data]
    assert sizes[L.weight_adjoint_id()] == 64 * 32 * ensemble * 4 and sizes[:2] == [x["array"].numel() for x in ref.data][:2]
    L.pass_init(m)
    w, wt = L.key_extract(m, "cem_weight_layer_dual")
    assert tuple(w.shape) == (ensemble, 64, 32) and tuple(wt.shape) == (64, 32, ensemble)
    assert w.data_ptr() == L.key_extract(m, "weights").data_ptr()
    L.key_extract(ref, "weights").copy_(w)
    xin = fill(L.key_extract(m, "input"), np.random.default_rng(5))
    L.key_extract(ref, "input").copy_(L.key_extract(m, "input"))
    L.graph_run_host(m, {"ensemble": ensemble})
    L.graph_run_host(ref, {"ensemble": ensemble})
    assert (host(L.key_extract(m, "output_probs")) == host(L.key_extract(ref, "output_probs"))).all()
    assert (host(L.key_extract(m, "output_indices")) == host(L.key_extract(ref, "output_indices"))).all()
    # apply_updates (ml/cem.spi:120-146) on the pair
    w0 = host(w).reshape(ensemble, -1).copy()
    rewards = dev(np.stack([np.arange(ensemble, dtype=np.float32), np.ones(ensemble, dtype=np.float32)], axis=1))
    mask = P.cem_update_rewards_mask(rewards)
    assert host(mask).tolist() == [0, 0, 0, 0, 1, 1, 1, 1] and (host(rewards) == 0).all()
    w2, wt2 = w.reshape(ensemble, -1), wt.reshape(-1, ensemble)
    P.grid_transpose(w2, wt2)
    assert (host(wt2) == w0.T).all()
    P.cem(wt2, mask, rng=(L._prim.CONSTANT_SEED, 0))
    norms = P.grid_map_reduce_map_2d("sqr", 0, "+", "sqrt", wt2)
    max_norm = float(P.reduce_max(norms))
    P.grid_transpose(wt2, w2)
    want_t = orow.cem_resample(w0.T.copy(), host(mask), ophilox.curand_normal_rows(64 * 32, ensemble), 0.1, 1.0)
    assert np.abs(host(w2) - want_t.T).max() < 2e-5 and (host(w2)[4:] == w0[4:]).all()
    assert abs(max_norm - np.sqrt((want_t.astype(np.float64) ** 2).sum(axis=1)).max()) < 1e-4


def test_other_heads_and_maps(L):
    announce("layers heads and maps")
    x = L.input("input", (Q, 8, 32))
    h = L.pipe(x, L.matmul((32, 32)))
    rm_node = L.regret_matching(h)
    g = L.pair(L.pair(L.argmax(L.tanh(h)), L.max(L.sigmoid(h))),
               L.pair(L.binarize(1000003, h), L.pair(L.discrete_sample(rm_node),
                                                    L.masked_regret_matching(5, L.copy(h)))))
    m = L.create_model(g)
    L.pass_init(m)
    rng = np.random.default_rng(2)
    xin = fill(L.key_extract(m, "input"), rng)
    (w,) = [host(t) for _, t, _ in L.extract_layers_(m, L.weight_id())]
    L.graph_run_host(m)
    (am, mx), (bits, (smp, mrm)) = L.graph_extract(m)
    hh = ogemm.gemm_abt(xin.reshape(-1, 32), w)
    # the product and the regret-matching probabilities as the kernels left them in the workspace: everything
    # computed FROM them (bits, sampled index) is compared bit for bit
    hk = host(L.graph_extract(L.Model(h, m.dims, m.data))).reshape(-1, 32)
    rmk = host(L.graph_extract(L.Model(rm_node, m.dims, m.data))).reshape(-1, 32)
    assert ogemm.rel_frobenius(hk, hh) < 1e-5
    assert ogemm.rel_frobenius(rmk, orow.regret_matching(hh)) < 1e-5
    assert (host(am).reshape(-1) == orow.argmax(np.tanh(hh))).all()
    assert np.abs(host(mx).reshape(-1) - (1 / (1 + np.exp(-hh))).max(axis=1)).max() < 1e-6
    assert (host(bits).reshape(-1).view(np.uint32) == orow.binarize(hk, 1000003)).all()
    u = ophilox.row_uniforms_layer(Q, 8, 32)
    picked = host(smp).reshape(-1)
    assert (picked == orow.discrete_sampling(rmk, u, order="wave")).all()
    assert (np.take_along_axis(rmk, picked[:, None].astype(np.int64), 1) > 0).all()
    assert ogemm.rel_frobenius(host(mrm).reshape(-1, 32), orow.masked_regret_matching(hh, 5)) < 1e-5


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_relu_mlp_graph_runs_fused(L, dtype):
    """A 16-bit matmul/relu chain with a masked sampling head is one sp_mlp_forward launch that
    writes only the head's outputs."""
    announce("layers fused graph " + dtype)
    g = L.pipe(L.input("input", (Q, 128, 32), dtype), L.matmul((32, 256)), L.relu, L.matmul((256, 256)), L.relu,
               L.matmul((256, 64)), L.masked_softmax_and_discrete_sample(3))
    m = L.create_model(g)
    assert L._fused_plan(m) is not None
    rng = np.random.default_rng(4)
    xin = fill(L.key_extract(m, "input"), rng)
    ws = [fill(t, rng, 1 / np.sqrt(t.shape[1])) for _, t, _ in L.extract_layers_(m, L.weight_id())]
    workspace = L.model_to_model_ptrs(m)[L.workspace_id()]
    first_hidden = L.graph_extract(L.Model(g.a.a.a.a.a, m.dims, m.data))
    first_hidden.fill_(7)
    L.graph_run_host(m)
    probs, idx = (host(t) for t in L.graph_extract(m))
    u = ophilox.row_uniforms_layer(Q, 128, 64)
    want, _, _ = olayers.mlp_forward(xin.reshape(-1, 32), ws, None, olayers.HEAD_SOFTMAX, u, None, 3)
    assert ogemm.rel_frobenius(probs.reshape(-1, 64), want) < 3e-3
    assert (idx.reshape(-1) == orow.discrete_sampling(probs.reshape(-1, 64), u)).all() and (idx < 3).all()
    assert (host(first_hidden.float()) == 7).all() and workspace.numel() > 0     # intermediates were never written
    # static weights: the same run on the packed kernel; new weights only count after weights_changed()
    for t in L.graph_extract(m):
        t.zero_()
    L.graph_run_host(m, static_weights=True)
    probs_s, idx_s = (host(t) for t in L.graph_extract(m))
    assert ogemm.rel_frobenius(probs_s, probs) < 2e-4 and (idx_s != idx).mean() < 1e-3
    first_w = [t for _, t, _ in L.extract_layers_(m, L.weight_id())][0]
    first_w.zero_()
    L.graph_run_host(m, static_weights=True)
    assert (host(L.graph_extract(m)[0]) == probs_s).all()                        # still the packed copy
    L.weights_changed(m)
    L.graph_run_host(m, static_weights=True)
    assert not (host(L.graph_extract(m)[0]) == probs_s).all()
    first_w.copy_(torch.from_numpy(ws[0]).to(first_w.dtype))
    L.weights_changed(m)
    with pytest.raises(Exception):
        L.graph_run_host(m, fuse=False)    # node by node the maps and row ops are f32-only


def test_main_body_writes_the_reference_files(L, tmp_path):
    announce("layers main_body")
    root = str(tmp_path) + "/"
    L.main_body(root)
    for i in range(1, 6):
        assert os.path.getsize(os.path.join(root, "test%d" % i, "layers.txt")) > 0
    t1 = open(os.path.join(root, "test1", "layers.txt")).read().splitlines()
    assert t1[0] == "---" and t1[4] == "Done initing." and len(t1) == 8 and t1[1].count("0.000000") == 16
    t3 = open(os.path.join(root, "test3", "layers.txt")).read()
    assert t3.startswith("Here are the weight matrices.\n[[") and t3.rstrip().endswith("====") and " ...]" in t3
    t5 = open(os.path.join(root, "test5", "layers.txt")).read()
    idx = np.array([int(v) for v in t5.replace("[", " ").replace("]", " ").replace(";", " ").split()])
    assert idx.size == 4 * Q * 64 and idx.min() >= 0 and idx.max() <= 10


@pytest.mark.parametrize("kind", ["nodes_f32", "fused_f16", "ensemble", "ensemble_loop"])
def test_replayed_runs_see_new_inputs_and_weights(L, kind):
    """graph_run_host records what its first run of a model launches and replays that afterwards.  A replay must read
    the tensors as they are NOW: inputs and weights are rewritten in place between runs, and every run is compared
    with the oracle and with the first (recording) run of a fresh model that holds the same values."""
    announce("layers replay " + kind)
    ensemble = 3

    def build():
        if kind == "fused_f16":
            g = L.pipe(L.input("input", (Q, 64, 32), "f16"), L.matmul((32, 256)), L.relu, L.matmul((256, 256)), L.relu,
                       L.matmul((256, 64)), L.masked_softmax_and_discrete_sample(5))
        elif kind == "nodes_f32":
            g = L.pipe(L.input("input", (Q, 64, 64)), L.matmul((64, 128)), L.relu, L.matmul((128, 64)), L.ln_l2, L.relu,
                       L.matmul((64, 64)), L.softmax_and_discrete_sample)
        else:
            out = L.pair(L.apply("ensemble", L.input("output_probs", (ensemble, Q, 64, 64))),
                         L.apply("ensemble", L.input("output_indices", (ensemble, Q, 64), "int")))
            x = L.pipe(L.input("input", (Q, 64, 64)), L.matmul_ensemble((ensemble, 64, 64)), L.relu,
                       L.matmul_ensemble((ensemble, 64, 64)))
            g = L.softmax_and_discrete_sample_(out, x)
        return L.create_model(g)

    sizes = {"ensemble": ensemble} if kind.startswith("ensemble") else {}
    kw = {"batched": False} if kind == "ensemble_loop" else {}

    def tensors(m):
        ws = L.key_extract_list(m, "weights") if sizes else [t for _, t, _ in L.extract_layers_(m, L.weight_id())]
        return [L.key_extract(m, "input")] + list(ws)

    def outputs(m):
        if sizes:
            return host(L.key_extract(m, "output_probs")), host(L.key_extract(m, "output_indices"))
        return tuple(host(t) for t in L.graph_extract(m, {}))

    m = build()
    previous = None
    for pass_ in range(3):
        rng = np.random.default_rng(100 + pass_)
        values = [(rng.standard_normal(tuple(t.shape)) * (1.0 if i == 0 else 0.1)).astype(np.float32)
                  for i, t in enumerate(tensors(m))]
        for t, v in zip(tensors(m), values):
            t.copy_(torch.from_numpy(v).to(t.dtype))
        L.graph_run_host(m, sizes, **kw)          # the first pass records, the second and third replay
        got = outputs(m)
        fresh = build()
        for t, v in zip(tensors(fresh), values):
            t.copy_(torch.from_numpy(v).to(t.dtype))
        L.graph_run_host(fresh, sizes, **kw)
        want = outputs(fresh)
        assert (got[0] == want[0]).all() and (got[1] == want[1]).all()
        assert np.abs(got[0].reshape(-1, got[0].shape[-1]).sum(axis=1) - 1).max() < 1e-4
        if previous is not None:
            assert not (got[0] == previous).all()
        previous = got[0]


@pytest.mark.parametrize("sampling", [False, True])
def test_leduc_policy_graph_runs_as_one_launch(L, sampling):
    """The graph of the reference's Leduc policy (game/leduc/model_cem.spi:55-63: input -> matmul_ensemble_with_adjoint
    (E, 128, 64) -> relu -> matmul_ensemble_with_adjoint (E, 64, 64) -> masked_regret_matching' 3 into the members'
    stacked output (or, second case, masked_softmax_and_discrete_sample' 3), paired with a table that computes nothing): `graph_run_host model {ensemble}` takes the fused
    ensemble kernel, and gives what the batched node-by-node pass gives (f32 bar: 1e-5) -- with a sampling head also the
    same draws per member: actions bit-exact given the policy and the stream."""
    from ml import _lib
    announce("layers leduc policy graph, sampling=%s" % sampling)
    ensemble, w = 8, 256
    probs = L.apply("ensemble", L.input("output_probs", (ensemble, Q, w, 64)))
    x = L.pipe(L.input("input", (Q, w, 128)), L.matmul_ensemble_with_adjoint((ensemble, 128, 64)), L.relu,
               L.matmul_ensemble_with_adjoint((ensemble, 64, 64)))
    if sampling:
        out = L.pair(probs, L.apply("ensemble", L.input("output_indices", (ensemble, Q, w), "int")))
        neural = L.masked_softmax_and_discrete_sample_(3, out, x)
    else:
        neural = L.masked_regret_matching_(3, probs, x)
    g = L.pair(neural, L.input("cem_table", (ensemble, 16, 4)))
    m = L.create_model(g)
    L.pass_init(m)
    fill(L.key_extract(m, "input"), np.random.default_rng(5))
    assert L._fused_ensemble_plan(m, "ensemble") is not None
    L.graph_run_host(m, {"ensemble": ensemble}, fuse=False)
    want_p = host(L.key_extract(m, "output_probs")).copy()
    want_i = host(L.key_extract(m, "output_indices")).copy() if sampling else None
    L.key_extract(m, "output_probs").fill_(7)
    for run in range(2):          # the second run replays the recorded launch
        L.graph_run_host(m, {"ensemble": ensemble})
        got_p = host(L.key_extract(m, "output_probs"))
        assert ogemm.rel_frobenius(got_p.reshape(-1, 64), want_p.reshape(-1, 64)) < 1e-5
        assert (got_p[..., 3:] == 0).all() and np.abs(got_p.sum(axis=-1) - 1).max() < 1e-5
        if sampling:
            got_i = host(L.key_extract(m, "output_indices"))
            assert (got_i != want_i).mean() < 1e-3          # (a policy one ulp apart can move a threshold across a draw)
            per_node = ophilox.draws_per_sampling_node(w, 64)
            for e in range(ensemble):
                u = ophilox.row_uniforms_layer(Q, w, 64, offset=e * per_node)
                assert (got_i[e].reshape(-1) == orow.discrete_sampling(got_p[e].reshape(-1, 64), u)).all()
    tape = m._tapes[(L._prim.CONSTANT_SEED, True, True, (("ensemble", ensemble),))][1]
    assert len(tape.calls) == 1 and tape.calls[0][0].__name__ == "sp_mlp_forward_ensemble"


def test_cfr_and_holdem_graphs_run_as_one_launch(L):
    """The other model graphs of the reference's agents: `input -> matmul_ensemble (E, 128, 128) -> binarize' 4096`
    (game/leduc/model_cfr.spi:56-61, game/nl_hu_holdem/model_cfr.spi:82-88) and `input -> matmul_ensemble_with_adjoint
    (E, 128, 64) -> masked_regret_matching' 3` (game/nl_hu_holdem/model_cem.spi:84-100), each paired with a table that
    computes nothing: one launch per run, results as the batched node-by-node pass gives them."""
    announce("layers cfr / holdem cem graphs")
    ensemble, w = 4, 256
    world = L.apply("ensemble", L.input("output_world_id", (ensemble, Q, w), "int"))
    g = L.pair(L.binarize_(1 << 12, world, L.pipe(L.input("input", (Q, w, 128)), L.matmul_ensemble((ensemble, 128, 128)))),
               L.input("cfr_table", (ensemble, 8, 4)))
    m = L.create_model(g)
    L.pass_init(m)
    fill(L.key_extract(m, "input"), np.random.default_rng(6))
    L.graph_run_host(m, {"ensemble": ensemble}, fuse=False)
    want = host(L.key_extract(m, "output_world_id")).copy()
    L.key_extract(m, "output_world_id").fill_(-1)
    for _ in range(2):
        L.graph_run_host(m, {"ensemble": ensemble})
        got = host(L.key_extract(m, "output_world_id"))
        assert (got != want).mean() < 1e-3 and (got >= 0).all() and (got < 4096).all()   # (signs of outputs next to zero)
    tape = m._tapes[(L._prim.CONSTANT_SEED, True, True, (("ensemble", ensemble),))][1]
    assert len(tape.calls) == 1 and tape.calls[0][0].__name__ == "sp_ensemble_binarize"

    probs = L.apply("ensemble", L.input("output_probs", (ensemble, Q, w, 64)))
    g = L.pair(L.masked_regret_matching_(3, probs, L.pipe(L.input("input", (Q, w, 128)),
                                                           L.matmul_ensemble_with_adjoint((ensemble, 128, 64)))),
               L.input("cem_table", (ensemble, 16, 4)))
    m = L.create_model(g)
    L.pass_init(m)
    fill(L.key_extract(m, "input"), np.random.default_rng(7))
    L.graph_run_host(m, {"ensemble": ensemble}, fuse=False)
    want_p = host(L.key_extract(m, "output_probs")).copy()
    L.key_extract(m, "output_probs").fill_(7)
    L.graph_run_host(m, {"ensemble": ensemble})
    got_p = host(L.key_extract(m, "output_probs"))
    assert ogemm.rel_frobenius(got_p.reshape(-1, 64), want_p.reshape(-1, 64)) < 1e-5 and (got_p[..., 3:] == 0).all()
    tape = m._tapes[(L._prim.CONSTANT_SEED, True, True, (("ensemble", ensemble),))][1]
    assert len(tape.calls) == 1 and tape.calls[0][0].__name__ == "sp_mlp_forward_ensemble"
