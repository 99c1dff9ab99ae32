"""Graph execution with MatMul / Gemm nodes routed to the BitNet provider.

The reference's `InferenceSession::execute_graph` (crates/ronn-api/src/session.rs:241-274) walks the
nodes in topological order, collects each node's inputs from a value cache and runs the node through
the ONNX operator registry; it never reaches an execution provider.  The patch under
`rust/patches/` adds `run_on_provider` to that loop.  This module is the same loop with the same
routing rule, over the Python face of the provider, so that the rule runs on a GPU:

* a `MatMul` or `Gemm` node goes to the provider when its second input is a graph initializer (a
  constant weight: the provider ternarises and caches that operand, which is only right for
  weights), both operands are 2-D, and - for Gemm - alpha = beta = 1 and transA = 0; transB = 1
  (the form a linear layer exports) is handled by transposing the constant once per node; Gemm's
  third input is added on the host;
* nodes that stand side by side in the graph with one shape and inputs that are already there - the
  q/k/v or gate/up projections of a token - are handed to `BitNetKernel.execute_group`, which runs
  them as one GPU launch in the decode regime (`ProviderRegistry::compile_subgraph`,
  crates/ronn-providers/src/registry.rs:237-266, would compile and run them one by one);
* every other node runs through a small host operator table (numpy), as the operator registry does
  in the reference; a node the provider declines is logged at warning level and runs there too.

Kernels are compiled once per node (or group of nodes) and kept, as `kernel_cache` does in the patch.
"""
import logging
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from .bitnet import BitNetExecutionProvider, Error, GraphNode, SubGraph, Tensor

log = logging.getLogger("ronn_amd.session")


def _attr(node: GraphNode, key: str, default):
    v = node.attributes.get(key, default)
    return default if v is None else v


def routable(node: GraphNode, initializers: Dict[str, np.ndarray], shapes: Dict[str, Tuple[int, ...]]) -> Optional[str]:
    """None when the node goes to the provider, else the reason it does not."""
    if node.op_type not in ("MatMul", "Gemm"):
        return "not a MatMul or Gemm node"
    if len(node.inputs) < 2 or (node.op_type == "MatMul" and len(node.inputs) != 2):
        return "needs two inputs"
    if node.inputs[1] not in initializers:
        return "second input is not a constant weight"
    if node.op_type == "Gemm":
        if float(_attr(node, "alpha", 1.0)) != 1.0 or float(_attr(node, "beta", 1.0)) != 1.0:
            return "Gemm with alpha or beta other than 1"
        if int(_attr(node, "transA", 0)) != 0:
            return "Gemm with transA"
    a, b = shapes.get(node.inputs[0]), shapes.get(node.inputs[1])
    if a is None or b is None or len(a) != 2 or len(b) != 2:
        return "operands are not 2-D"
    return None


def _weight_shape(node: GraphNode, b_shape):
    trans_b = node.op_type == "Gemm" and int(_attr(node, "transB", 0)) != 0
    return (b_shape[1], b_shape[0]) if trans_b else tuple(b_shape)


@dataclass
class Step:
    """One step of the plan: `nodes` run together; kind is "group" (several nodes, one provider call),
    "provider" (one node, one provider call) or "host" (the operator table), with the reason."""
    kind: str
    nodes: List[GraphNode]
    reason: str = ""


def plan_routing(nodes: Sequence[GraphNode], initializers: Dict[str, np.ndarray],
                 input_shapes: Dict[str, Tuple[int, ...]]) -> List[Step]:
    """Which nodes go where, from shapes alone (needs no device).  Nodes are in topological order.
    A group is a run of consecutive routable nodes with one [m,k] x [k,n] shape whose inputs do not
    come out of the run itself."""
    shapes = {k: tuple(v.shape) for k, v in initializers.items()}
    shapes.update({k: tuple(v) for k, v in input_shapes.items()})
    steps: List[Step] = []
    i = 0
    nodes = list(nodes)
    while i < len(nodes):
        node = nodes[i]
        why = routable(node, initializers, shapes)
        if why is not None:
            steps.append(Step("host", [node], why))
            _infer(node, shapes)
            i += 1
            continue
        sig = (shapes[node.inputs[0]], _weight_shape(node, shapes[node.inputs[1]]))
        run, produced = [node], set(node.outputs)
        j = i + 1
        while j < len(nodes):
            nxt = nodes[j]
            if routable(nxt, initializers, shapes) is not None or nxt.inputs[0] in produced:
                break
            if (shapes[nxt.inputs[0]], _weight_shape(nxt, shapes[nxt.inputs[1]])) != sig:
                break
            run.append(nxt)
            produced.update(nxt.outputs)
            j += 1
        steps.append(Step("group" if len(run) > 1 else "provider", run))
        for n in run:
            _infer(n, shapes)
        i = j
    return steps


def _infer(node: GraphNode, shapes):
    """Output shape of the few operators the table below knows (enough to plan a graph)."""
    ins = [shapes.get(n) for n in node.inputs]
    out = None
    if node.op_type in ("MatMul", "Gemm") and ins[0] is not None and ins[1] is not None and len(ins[0]) == 2 and len(ins[1]) == 2:
        a, b = ins[0], ins[1]
        if node.op_type == "Gemm":
            if int(_attr(node, "transA", 0)):
                a = (a[1], a[0])
            if int(_attr(node, "transB", 0)):
                b = (b[1], b[0])
        out = (a[0], b[1])
    elif node.op_type in ("Add", "Sub", "Mul") and ins[0] is not None and ins[1] is not None:
        out = tuple(np.broadcast_shapes(ins[0], ins[1]))
    elif node.op_type in ("Relu", "Sigmoid") and ins[0] is not None:
        out = ins[0]
    for name in node.outputs:
        shapes[name] = out


def _host_op(node: GraphNode, ins: List[np.ndarray]) -> List[np.ndarray]:
    """The host operator table: what crates/ronn-onnx/src/ops/ gives these nodes (f32)."""
    op = node.op_type
    if op == "MatMul":
        return [(ins[0] @ ins[1]).astype(np.float32)]
    if op == "Gemm":
        a = ins[0].T if int(_attr(node, "transA", 0)) else ins[0]
        b = ins[1].T if int(_attr(node, "transB", 0)) else ins[1]
        r = (a @ b).astype(np.float32) * np.float32(_attr(node, "alpha", 1.0))
        if len(ins) > 2:
            r = r + ins[2] * np.float32(_attr(node, "beta", 1.0))
        return [r.astype(np.float32)]
    if op == "Add":
        return [(ins[0] + ins[1]).astype(np.float32)]
    if op == "Sub":
        return [(ins[0] - ins[1]).astype(np.float32)]
    if op == "Mul":
        return [(ins[0] * ins[1]).astype(np.float32)]
    if op == "Relu":
        return [np.maximum(ins[0], 0).astype(np.float32)]
    if op == "Sigmoid":
        return [(1.0 / (1.0 + np.exp(-ins[0]))).astype(np.float32)]
    raise Error("Operator %s not supported" % op)   # session.rs:256-258


class RoutedSession:
    """`InferenceSession::run` with the BitNet provider behind MatMul / Gemm nodes."""

    def __init__(self, provider: BitNetExecutionProvider, nodes: Sequence[GraphNode],
                 initializers: Dict[str, np.ndarray], outputs: Sequence[str]):
        self.provider = provider
        self.nodes = list(nodes)
        self.initializers = {k: np.ascontiguousarray(v, dtype=np.float32) for k, v in initializers.items()}
        self.outputs = list(outputs)
        self.kernel_cache = {}     # node ids of a step -> compiled kernel
        self.weight_cache = {}     # node id -> the constant as [k, n] (transposed once when transB = 1)
        self.routed_nodes = 0      # nodes that ran on the provider in the last run()
        self.provider_calls = 0    # execute() / execute_group() calls of the last run()
        self.gpu_launches = 0      # matmul launches those calls issued (groups report theirs)
        self.host_nodes = 0

    def _weight(self, node: GraphNode) -> np.ndarray:
        w = self.weight_cache.get(node.id)
        if w is None:
            w = self.initializers[node.inputs[1]]
            if node.op_type == "Gemm" and int(_attr(node, "transB", 0)):
                w = np.ascontiguousarray(w.T)
            self.weight_cache[node.id] = w
        return w

    def _kernel(self, step: Step):
        key = tuple(n.id for n in step.nodes)
        k = self.kernel_cache.get(key)
        if k is None:
            first = step.nodes[0]
            k = self.provider.compile_subgraph(SubGraph(nodes=[first], inputs=list(first.inputs),
                                                        outputs=list(first.outputs)))
            self.kernel_cache[key] = k
        return k

    def run(self, inputs: Dict[str, np.ndarray]) -> Dict[str, np.ndarray]:
        values = dict(self.initializers)                                    # session.rs:174-177
        values.update({k: np.ascontiguousarray(v, dtype=np.float32) for k, v in inputs.items()})
        self.routed_nodes = self.provider_calls = self.gpu_launches = self.host_nodes = 0
        steps = plan_routing(self.nodes, self.initializers, {k: v.shape for k, v in inputs.items()})
        for step in steps:
            done = False
            if step.kind != "host":
                try:
                    kernel = self._kernel(step)
                    pairs = []
                    for n in step.nodes:
                        a, w = values[n.inputs[0]], self._weight(n)
                        pairs += [Tensor.from_data(a, list(a.shape)), Tensor.from_data(w, list(w.shape))]
                    if step.kind == "group":
                        outs = kernel.execute_group(pairs)
                        self.gpu_launches += kernel.last_group_launches
                    else:
                        outs = kernel.execute(pairs)
                        self.gpu_launches += 1
                    self.provider_calls += 1
                    for n, o in zip(step.nodes, outs):
                        r = o.numpy()
                        if n.op_type == "Gemm" and len(n.inputs) > 2:
                            r = (r + values[n.inputs[2]]).astype(np.float32)   # Y = A * B + C on the host
                        values[n.outputs[0]] = r
                    self.routed_nodes += len(step.nodes)
                    done = True
                except Error as e:
                    log.warning("BitNet provider declined node(s) %s: %s; using the host operator",
                                [n.id for n in step.nodes], e)
            if not done:
                for n in step.nodes:
                    ins = [values[name] for name in n.inputs if name in values]
                    for name, r in zip(n.outputs, _host_op(n, ins)):
                        values[name] = r
                    self.host_nodes += 1
        missing = [o for o in self.outputs if o not in values]
        if missing:
            raise Error("graph outputs were never produced: %s" % missing)
        return {o: values[o] for o in self.outputs}
