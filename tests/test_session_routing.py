"""Graph routing: which nodes of a graph go to the BitNet provider (crates/ronn-api/src/session.rs:241-274
with the routing of rust/patches/route-matmul-gemm-to-bitnet-provider.patch), planned on the CPU and run on
a GPU through the Python face of the provider."""
import numpy as np
import pytest

from ronn_amd.bitnet import GraphNode
from ronn_amd.session import plan_routing


def projection_graph(k=64, n=48, n_out=32):
    rng = np.random.default_rng(5)
    init = {"Wq": rng.normal(0, 0.02, (k, n)).astype(np.float32),
            "Wk": rng.normal(0, 0.02, (k, n)).astype(np.float32),
            "Wv": rng.normal(0, 0.02, (k, n)).astype(np.float32),
            "Wo_t": rng.normal(0, 0.02, (n_out, n)).astype(np.float32),     # stored [n_out, n]: Gemm with transB = 1
            "bo": rng.normal(0, 0.1, (n_out,)).astype(np.float32),
            "Ws": rng.normal(0, 0.02, (n, n)).astype(np.float32)}
    nodes = [GraphNode(0, "MatMul", inputs=["x", "Wq"], outputs=["q"]),
             GraphNode(1, "MatMul", inputs=["x", "Wk"], outputs=["k"]),
             GraphNode(2, "MatMul", inputs=["x", "Wv"], outputs=["v"]),
             GraphNode(3, "Mul", inputs=["q", "k"], outputs=["qk"]),
             GraphNode(4, "Add", inputs=["qk", "v"], outputs=["h"]),
             GraphNode(5, "Relu", inputs=["h"], outputs=["hr"]),
             GraphNode(6, "Gemm", {"transB": 1}, ["hr", "Wo_t", "bo"], ["o"]),
             GraphNode(7, "MatMul", inputs=["hr", "h"], outputs=["never"]),  # two run-time tensors
             GraphNode(8, "Gemm", {"alpha": 2.0}, ["hr", "Ws"], ["scaled"])]
    return nodes, init


def test_routing_plan_needs_no_device():
    nodes, init = projection_graph()
    nodes = [n for n in nodes if n.id != 7]
    steps = plan_routing(nodes, init, {"x": (1, 64)})
    kinds = [(s.kind, [n.id for n in s.nodes]) for s in steps]
    assert kinds == [("group", [0, 1, 2]), ("host", [3]), ("host", [4]), ("host", [5]), ("provider", [6]), ("host", [8])]
    assert steps[-1].reason == "Gemm with alpha or beta other than 1"
    # a product of two run-time tensors is never routed: the provider ternarises its second operand
    n7 = GraphNode(7, "MatMul", inputs=["q", "k"], outputs=["s"])
    assert plan_routing([nodes[0], nodes[1], n7], init, {"x": (4, 64)})[-1].reason == "second input is not a constant weight"
    # a node that consumes an output of the run does not join it, and another shape starts a new step
    chain = [GraphNode(0, "MatMul", inputs=["x", "Ws"], outputs=["a"]), GraphNode(1, "MatMul", inputs=["a", "Ws"], outputs=["b"])]
    assert [s.kind for s in plan_routing(chain, init, {"x": (1, 48)})] == ["provider", "provider"]
    mixed = [GraphNode(0, "MatMul", inputs=["x", "Wq"], outputs=["a"]), GraphNode(1, "Gemm", {"transB": 1}, ["x", "Wo_t"], ["b"])]
    init2 = dict(init, Wo_t=init["Wo_t"][:, :64] if init["Wo_t"].shape[1] >= 64 else np.zeros((32, 64), np.float32))
    assert [s.kind for s in plan_routing(mixed, init2, {"x": (1, 64)})] == ["provider", "provider"]


@pytest.mark.gpu
def test_session_routes_projections_to_the_provider_and_the_rest_to_the_host():
    from oracle import oracle as O
    from ronn_amd.bitnet import create_bitnet_provider
    from ronn_amd.session import RoutedSession
    from util import same_bits
    nodes, init = projection_graph()
    nodes = [n for n in nodes if n.id != 7]
    sess = RoutedSession(create_bitnet_provider(), nodes, init, ["q", "k", "v", "o", "scaled"])
    for m in (1, 5):
        x = np.random.default_rng(m).normal(0, 1, (m, 64)).astype(np.float32)
        out = sess.run({"x": x})
        # q/k/v: one provider call; in the decode regime one GPU launch for the three nodes
        assert sess.routed_nodes == 4 and sess.provider_calls == 2 and sess.host_nodes == 4
        assert sess.gpu_launches == (2 if m == 1 else 4)
        q, k, v = (O.execute_ternary(x, init[w])[0] for w in ("Wq", "Wk", "Wv"))
        assert same_bits(out["q"], q) and same_bits(out["k"], k) and same_bits(out["v"], v)
        hr = np.maximum((q * k).astype(np.float32) + v, 0).astype(np.float32)
        want_o = (O.execute_ternary(hr, np.ascontiguousarray(init["Wo_t"].T))[0] + init["bo"]).astype(np.float32)
        assert same_bits(out["o"], want_o)
        assert np.allclose(out["scaled"], 2.0 * (hr @ init["Ws"]), rtol=1e-5, atol=1e-6)      # host path, f32
    assert len(sess.kernel_cache) == 2 and list(sess.weight_cache) == [0, 1, 2, 6]
