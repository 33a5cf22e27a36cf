"""The layer-graph front end without a GPU: dimensions, the reference's asserts, and the byte-arena
layout.  The arena sizes are the ones the reference's generated module allocates for its own test
graphs with 24 blocks per grid (`cp.empty(N, dtype=cp.uint8)` at ml/layers.py:4736-4737, 5194-5195,
5548-5549, 6085-6086, 6640-6641: workspace, then weights; the adjoint arena is empty)."""
import pytest
import torch

from ml import layers as L


@pytest.fixture(autouse=True)
def blocks_24():
    L.set_blocks_per_grid(24)
    yield
    L.set_blocks_per_grid(24)


def sizes(graph):
    return [p["size"] for p in L.pass_calculate_partitions(graph, {})]


def tanh_mlp(k):
    return L.pipe(L.input("input", (24, 1, k)), L.matmul((k, 4)), L.tanh, L.matmul((4, 4)), L.tanh, L.matmul((4, 2)),
                  L.tanh)


def graph_of_test3():
    return L.pipe(L.input("input", (24, 64, 64)), L.matmul((64, 64)), L.ln_l2, L.relu, L.matmul((64, 64)), L.ln_l2,
                  L.relu, L.matmul((64, 64)), L.softmax_and_discrete_sample)


def ensemble_graph(e, deep, size=None):
    out = L.pair(L.apply("ensemble", L.input("output_probs", (e, 24, 64, 64))),
                 L.apply("ensemble", L.input("output_indices", (e, 24, 64), "int")))
    x = L.pipe(L.input("input", (24, 64, 64)), L.matmul_ensemble((e, 64, 64)))
    if deep:
        x = L.pipe(x, L.ln_l2, L.relu, L.matmul_ensemble((e, 64, 64)), L.ln_l2, L.relu, L.matmul_ensemble((e, 64, 64)))
    return L.softmax_and_discrete_sample_(out, x) if size is None else \
        L.masked_softmax_and_discrete_sample_(size, out, x)


def test_arena_sizes_match_the_reference():
    assert sizes(tanh_mlp(4)) == [160, 2304, 0]                    # layers test1
    assert sizes(tanh_mlp(2)) == [128, 2112, 0]                    # layers test2
    assert sizes(graph_of_test3()) == [49152, 3545088, 0]             # layers test3
    assert sizes(ensemble_graph(16, True)) == [786432, 9535488, 0]  # layers test4
    assert sizes(ensemble_graph(4, False, 11)) == [65536, 2383872, 0]  # layers test5


def test_offsets_are_depth_first_and_16_byte_aligned():
    g = L.pipe(L.input("input", (24, 1, 3)), L.matmul((3, 5)), L.tanh)     # 12- and 20-byte rows: padding appears
    parts = L.pass_calculate_partitions(g, {})
    ws = sorted((o.offset, o.spec.dim) for o in parts[L.workspace_id()]["partition"].values())
    assert [d for _, d in ws] == [(24, 1, 3), (24, 1, 5), (24, 1, 5)]
    assert [o for o, _ in ws] == [0, 288, 288 + 480]
    assert all(o % 16 == 0 for o, _ in ws)
    g2 = L.pipe(L.input("input", (24, 1, 1)), L.matmul((1, 1)), L.matmul((1, 1)))
    parts = L.pass_calculate_partitions(g2, {})
    assert sorted(o.offset for o in parts[L.weight_id()]["partition"].values()) == [0, 16]   # 4-byte weights, 16 apart
    assert parts[L.weight_id()]["size"] == 20                                            # the end is not padded


def test_dimension_asserts_are_the_reference_ones():
    with pytest.raises(AssertionError, match="batch dimension in the matmul node"):
        L.get_dim({}, L.pipe(L.input("input", (7, 4, 4)), L.matmul((4, 4))))
    with pytest.raises(AssertionError, match="inner dimensions of the matrix multiplication"):
        L.get_dim({}, L.BlockMatmul(L.input("input", (24, 4, 4)), L.weight((8, 5))))
    with pytest.raises(AssertionError, match="dimensions of the first output"):
        L.get_dim_pair({}, L.softmax_and_discrete_sample_(
            L.pair(L.input_((24, 4, 8)), L.input_((24, 4), "int")), L.input("input", (24, 4, 4))))
    d = L.get_dim_pair({}, graph_of_test3())
    assert d[0].dim == (24, 64, 64) and d[1].dim == (24, 64) and d[1].dtype == torch.int32
    assert L.get_dim({}, L.argmax(L.input("x", (24, 8, 12)))).dim == (24, 8)
    assert L.get_dim({}, L.binarize(7, L.input("x", (24, 8, 12)))).dim == (24, 8)


def test_extract_and_model_ptrs_on_host_memory():
    g = ensemble_graph(4, False, 11)
    m = L.create_model(g, device="cpu")
    for x in m.data:
        x["array"].zero_()
    w = L.key_extract(m, "weights")
    assert w.shape == (4, 64, 64) and w.dtype == torch.float32
    w[2, 1, 3] = 5.0
    probs, idx = L.graph_extract(m, {"ensemble": 3})
    assert probs.shape == (24, 64, 64) and idx.shape == (24, 64) and idx.dtype == torch.int32
    idx[0, 0] = 77
    assert L.key_extract(m, "output_indices")[3, 0, 0] == 77
    with pytest.raises(KeyError, match="missing .scalar. key"):
        L.graph_extract(m, {})
    with pytest.raises(KeyError, match="Cannot find the input tensor"):
        L.key_extract(m, "nothing")
    # the same arenas seen through a second model built around the pointers
    m2 = L.model_ptrs_to_model(g, L.model_to_model_ptrs(m))
    assert L.key_extract(m2, "weights")[2, 1, 3] == 5.0
    with pytest.raises(AssertionError, match="length of the partition"):
        L.model_ptrs_to_model(g, tuple(torch.empty(8, dtype=torch.uint8) for _ in range(3)))
    assert [sid for sid, _, _ in L.extract_layers(m)] == [1, 0, 1, 1]
    L.set_random_seed(1, device="cpu")
    L.pass_init(m)
    w = L.key_extract(m, "weights")
    assert abs(float(w.std()) - 0.1) < 0.01 and L.key_extract(m, "input").abs().sum() == 0


def test_printing_uses_the_golden_text_format():
    m = L.create_model(tanh_mlp(4), device="cpu")
    for x in m.data:
        x["array"].zero_()
    lines = []
    L.print_weights(m, lines.append)
    # the first three lines of the reference's layers/test1/layers.txt after "---"
    row = "[0.000000; 0.000000; 0.000000; 0.000000]"
    assert lines == ["[" + "; ".join([row] * 4) + "]"] * 2 + ["[" + "; ".join([row] * 2) + "]"]


def test_fused_plan_takes_only_the_shapes_the_fused_kernel_runs():
    """A 16-bit relu stack with a sampling head is planned as one fused launch only for the widths the fused
    kernel accepts (input a multiple of 16, hidden widths multiples of 32, nothing above 256, head <= 64)."""
    def stack(dims, dtype="f16"):
        x = L.input("input", (24, 16, dims[0]), dtype)
        for i, (k, n) in enumerate(zip(dims[:-1], dims[1:])):
            x = L.matmul((k, n), x)
            if i + 2 < len(dims):
                x = L.relu(x)
        return L.create_model(L.masked_softmax_and_discrete_sample(3, x), device="cpu")

    assert L._fused_plan(stack([32, 256, 256, 64])) is not None
    assert L._fused_plan(stack([32, 64, 3 * 32, 16])) is not None
    assert L._fused_plan(stack([32, 48, 16])) is None          # hidden width not a multiple of 32
    assert L._fused_plan(stack([32, 256, 128])) is None        # head wider than 64
    assert L._fused_plan(stack([24, 256, 64])) is None         # input width not a multiple of 16
    assert L._fused_plan(stack([32, 512, 64])) is None         # wider than 256
    assert L._fused_plan(stack([32, 256, 64], "float")) is None   # f32 graphs run node by node


def test_ensemble_with_adjoint_places_the_dual_in_the_adjoint_arena():
    """`matmul_ensemble_with_adjoint` (ml/layers.spi:472-479): weights (E, out, in) in the weights arena, their dual
    ((out, in), E) in the third arena, both reachable under "cem_weight_layer_dual", the product as matmul_ensemble's."""
    e, k, n = 4, 32, 64
    x = L.pipe(L.input("input", (24, 64, k)), L.matmul_ensemble_with_adjoint((e, k, n)))
    g = L.softmax_and_discrete_sample(x)
    plain = L.softmax_and_discrete_sample(L.pipe(L.input("input", (24, 64, k)), L.matmul_ensemble((e, k, n))))
    assert sizes(g) == sizes(plain)[:2] + [n * k * e * 4]
    m = L.create_model(g, device="cpu")
    w, wt = L.key_extract(m, "cem_weight_layer_dual")
    assert tuple(w.shape) == (e, n, k) and tuple(wt.shape) == (n, k, e)
    assert w.data_ptr() == L.key_extract(m, "weights").data_ptr()
    assert wt.data_ptr() == L.model_to_model_ptrs(m)[L.weight_adjoint_id()].data_ptr()
    assert L.get_dim({}, x).dim == (24, 64, n)
