"""Op graph, clean-up passes and per-element fusion into clusters.

Host-side mirror of src/op.rs and src/graph.rs: the structure the device
backend receives is `Graph.clusters_sorted`, a topologically ordered list of
`Cluster`s (one kernel descriptor plus the op nodes it reads and writes).

The graph container follows petgraph's `StableDiGraph` conventions that the
reference's results depend on: node ids are never reused, a node's edge list
is walked most-recent-first, and `Topo` pops its work list LIFO.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

from .kernel import (
    FillKernel,
    Literal,
    MatMulKernel,
    PeBinary,
    PeCoord,
    PeGather,
    PeLiteral,
    PeLoad,
    PeRand,
    PeSelect,
    PeUnary,
    PerElementKernel,
    ReduceKernel,
    ScatterAddKernel,
    UnpadKernel,
    WindowsToImageKernel,
)
from .shape import Shape, View

MAX_OP_ARGS = 4  # src/op.rs:72


@dataclass(frozen=True)
class Op:
    """src/op.rs:82-97. `kind` names the variant; `a`, `b` carry its fields:
    Input/Output(a=parameter), Literal(a=Literal), Coord, Rand(a=uid),
    Unary(a=name), Binary(a=name), Select(a=mode), MatMul(a=output_mode),
    Reduce(a=name, b=axis), Unpad(a=axis, b=pad), WindowsToImage(a=(sw,sh)),
    Gather(a=axis), ScatterAdd(a=axis)."""

    kind: str
    a: object = None
    b: object = None

    def is_per_element(self) -> bool:  # src/op.rs:114-119
        return self.kind in ("Unary", "Binary", "Select", "Gather")

    def is_gather_arg(self, arg: int) -> bool:  # src/op.rs:121-126
        return self.kind == "Gather" and arg == 0

    def can_reshape(self) -> bool:  # src/op.rs:128-130
        return self.kind not in ("Coord", "Rand", "Gather")

    def can_merge(self) -> bool:  # src/op.rs:132-134
        return self.kind not in ("Input", "Output")

    def is_builtin(self) -> bool:
        return self.kind in ("Coord", "Rand")

    def __str__(self):
        if self.kind in ("Unary", "Binary"):
            return str(self.a)
        if self.kind == "Select":
            return f"Select{self.a}"
        if self.kind == "Reduce":
            return f"Reduce{self.a}({self.b})"
        if self.kind == "Literal":
            return repr(self.a)
        return self.kind


MOV = Op("Unary", "Mov")


@dataclass
class OpNode:  # src/op.rs:162-168
    colour: int
    shape: Shape
    op: Op
    cluster_id: Optional[int] = None


@dataclass
class OpEdge:  # src/op.rs:170-180
    src: int
    dst: int
    arg: int
    view: View

    def is_per_element(self, dst_op: Op) -> bool:
        return not dst_op.is_gather_arg(self.arg) and self.view.is_contiguous()


class OpGraph:
    """Directed multigraph with stable node/edge ids."""

    def __init__(self):
        self.nodes: Dict[int, OpNode] = {}
        self.edges: Dict[int, OpEdge] = {}
        self._out: Dict[int, List[int]] = {}
        self._in: Dict[int, List[int]] = {}
        self._next_node = 0
        self._next_edge = 0

    def clone(self) -> "OpGraph":
        g = OpGraph()
        g.nodes = {i: OpNode(n.colour, n.shape, n.op, n.cluster_id) for i, n in self.nodes.items()}
        g.edges = {i: OpEdge(e.src, e.dst, e.arg, e.view) for i, e in self.edges.items()}
        g._out = {i: list(v) for i, v in self._out.items()}
        g._in = {i: list(v) for i, v in self._in.items()}
        g._next_node, g._next_edge = self._next_node, self._next_edge
        return g

    # -- construction ------------------------------------------------------
    def add_node(self, node: OpNode) -> int:
        nid = self._next_node
        self._next_node += 1
        self.nodes[nid] = node
        self._out[nid] = []
        self._in[nid] = []
        return nid

    def add_edge(self, src: int, dst: int, arg: int, view: View) -> int:
        eid = self._next_edge
        self._next_edge += 1
        self.edges[eid] = OpEdge(src, dst, arg, view)
        self._out[src].append(eid)
        self._in[dst].append(eid)
        return eid

    def new_node(self, colour: int, shape, op: Op, inputs=()) -> int:
        """src/op.rs:192-219: edges from `inputs` get identity views."""
        nid = self.add_node(OpNode(colour, Shape(shape), op))
        for arg, src in enumerate(inputs):
            self.add_edge(src, nid, arg, self.nodes[src].shape.identity_view())
        return nid

    def remove_edge(self, eid: int):
        e = self.edges.pop(eid)
        self._out[e.src].remove(eid)
        self._in[e.dst].remove(eid)

    def remove_node(self, nid: int):
        for eid in list(self._out[nid]) + list(self._in[nid]):
            if eid in self.edges:
                self.remove_edge(eid)
        del self.nodes[nid], self._out[nid], self._in[nid]

    # -- queries -----------------------------------------------------------
    def node_bound(self) -> int:
        return self._next_node

    def in_edges(self, nid: int) -> List[int]:
        return list(reversed(self._in[nid]))

    def out_edges(self, nid: int) -> List[int]:
        return list(reversed(self._out[nid]))

    def predecessors(self, nid: int) -> List[int]:
        return [self.edges[e].src for e in self.in_edges(nid)]

    def successors(self, nid: int) -> List[int]:
        return [self.edges[e].dst for e in self.out_edges(nid)]

    def arg_edge_ids(self, nid: int) -> List[int]:
        """Incoming edges ordered by argument slot (src/graph.rs:19-29)."""
        by_arg: Dict[int, int] = {}
        for eid in self._in[nid]:
            arg = self.edges[eid].arg
            assert arg not in by_arg, "two edges feed the same argument"
            by_arg[arg] = eid
        n = max(by_arg) + 1 if by_arg else 0
        return [by_arg[i] for i in range(n)]

    def topo_order(self) -> List[int]:
        """petgraph `Topo`: seeds are the nodes without inputs in id order, the
        work list is a stack, and a successor becomes ready once all of its
        predecessors have been emitted."""
        stack = [n for n in sorted(self.nodes) if not self._in[n]]
        done = set()
        order = []
        while stack:
            n = stack.pop()
            if n in done:
                continue
            done.add(n)
            order.append(n)
            for m in self.successors(n):
                if m not in done and all(p in done for p in self.predecessors(m)):
                    stack.append(m)
        return order


@dataclass(frozen=True)
class ArgSource:  # src/graph.rs:31-36
    node_id: int
    is_gather: bool
    view: View


def get_arg_sources(ops: OpGraph, nid: int) -> List[ArgSource]:
    out = []
    for eid in ops.arg_edge_ids(nid):
        e = ops.edges[eid]
        out.append(ArgSource(e.src, ops.nodes[e.dst].op.is_gather_arg(e.arg), e.view))
    return out


@dataclass
class ClusterOutput:  # src/graph.rs:56-82
    node_id: int
    copy_from: Optional[int] = None  # InitialState::CopyFrom(node) / Undefined


@dataclass
class Cluster:  # src/graph.rs:84-89
    kernel: object
    inputs: List[int] = field(default_factory=list)
    outputs: List[ClusterOutput] = field(default_factory=list)


class Graph:
    """src/graph.rs:102-139: runs the passes in the reference's order and
    leaves `clusters` / `clusters_sorted` for the executor."""

    def __init__(self, ops: OpGraph):
        self.ops = ops
        self.ops_sorted: List[int] = []
        self.clusters: Dict[int, Cluster] = {}
        self.clusters_sorted: List[int] = []

        self._rebuild_ordering()
        self._eliminate_dead_code()
        self._rebuild_ordering()
        self._eliminate_moves()
        self._rebuild_ordering()
        self._simplify_arithmetic()
        self._rebuild_ordering()
        self._eliminate_common_subgraphs()
        self._rebuild_ordering()
        self._make_built_ins_and_literals_unique()
        self._rebuild_ordering()
        self._build_clusters()

    # -- passes ------------------------------------------------------------
    def _rebuild_ordering(self):
        self.ops_sorted = self.ops.topo_order()
        assert len(self.ops_sorted) == len(self.ops.nodes), "op graph has a cycle"

    def _eliminate_dead_code(self):
        """Keep what reaches an Output (src/graph.rs:150-165)."""
        ops = self.ops
        live = {n for n, node in ops.nodes.items() if node.op.kind == "Output"}
        for n in reversed(self.ops_sorted):
            if n in live:
                live.update(ops.predecessors(n))
        for n in [n for n in ops.nodes if n not in live]:
            ops.remove_node(n)

    def _eliminate_moves(self):
        """Fold Mov nodes into the views of the edges around them where the
        views compose (src/graph.rs:255-301)."""
        ops = self.ops
        for nid in self.ops_sorted:
            if nid not in ops.nodes or ops.nodes[nid].op != MOV:
                continue
            in_edges = ops.in_edges(nid)
            assert len(in_edges) == 1, "Mov without exactly one source (gradient never accumulated?)"
            in_eid = in_edges[0]
            in_edge = ops.edges[in_eid]
            in_node = in_edge.src
            match = View.try_from_reshape(in_edge.view.output_shape, ops.nodes[nid].shape)
            if match is not None:
                in_edge.view = in_edge.view.through(match, False)
            can_reshape = ops.nodes[in_node].op.can_reshape()
            out_eids = ops.out_edges(nid)
            ok = all(
                ops.nodes[ops.edges[e].dst].op.kind != "Output"
                and in_edge.view.can_view_through(ops.edges[e].view, can_reshape)
                for e in out_eids
            )
            if ok:
                for e in out_eids:
                    oe = ops.edges[e]
                    assert in_edge.arg == 0
                    ops.add_edge(in_node, oe.dst, oe.arg, in_edge.view.through(oe.view, can_reshape))
                ops.remove_node(nid)

    def _simplify_arithmetic(self):
        """x*1, x+0 (and the u32 forms) become Mov (src/graph.rs:221-253)."""
        ops = self.ops
        identity = {
            "Mul": Literal.f32(1.0),
            "Add": Literal.f32(0.0),
            "UMul": Literal.u32(1),
            "UAdd": Literal.u32(0),
        }
        mov_added = False
        for nid in self.ops_sorted:
            node = ops.nodes[nid]
            if node.op.kind != "Binary" or node.op.a not in identity:
                continue
            skip = Op("Literal", identity[node.op.a])
            arg_eids = ops.arg_edge_ids(nid)
            skip_eid = next((e for e in arg_eids if ops.nodes[ops.edges[e].src].op == skip), None)
            if skip_eid is None:
                continue
            for e in arg_eids:
                if e == skip_eid:
                    ops.remove_edge(e)
                else:
                    node.op = MOV
                    ops.edges[e].arg = 0
            mov_added = True
        if mov_added:
            self._eliminate_moves()

    def _eliminate_common_subgraphs(self):
        """src/graph.rs:167-203."""
        ops = self.ops
        seen: Dict[tuple, int] = {}
        for nid in self.ops_sorted:
            if nid not in ops.nodes:
                continue
            node = ops.nodes[nid]
            if not node.op.can_merge():
                continue
            key = (tuple(get_arg_sources(ops, nid)), node.shape, node.op)
            other = seen.get(key)
            if other is None:
                seen[key] = nid
                continue
            for e in ops.out_edges(nid):
                oe = ops.edges[e]
                ops.add_edge(other, oe.dst, oe.arg, oe.view)
            ops.remove_node(nid)

    def _make_built_ins_and_literals_unique(self):
        """One private copy per consumer, so they can be inlined into every
        cluster that uses them (src/graph.rs:205-219)."""
        ops = self.ops
        for nid in self.ops_sorted:
            node = ops.nodes[nid]
            if node.op.kind == "Literal" or node.op.is_builtin():
                for e in ops.out_edges(nid):
                    oe = ops.edges[e]
                    new_id = ops.add_node(OpNode(node.colour, node.shape, node.op, node.cluster_id))
                    ops.add_edge(new_id, oe.dst, oe.arg, oe.view)
                ops.remove_node(nid)

    # -- reachability helpers (src/graph.rs:303-341) -------------------------
    def _any_predecessor(self, roots, pred) -> bool:
        ops = self.ops
        marked = set(roots)
        for nid in reversed(self.ops_sorted):
            if any(s in marked for s in ops.successors(nid)):
                marked.add(nid)
                if pred(nid):
                    return True
        return False

    def _any_successor(self, roots, pred) -> bool:
        ops = self.ops
        marked = set(roots)
        for nid in self.ops_sorted:
            if any(p in marked for p in ops.predecessors(nid)):
                marked.add(nid)
                if pred(nid):
                    return True
        return False

    # -- clustering (src/graph.rs:344-654) -----------------------------------
    def _build_clusters(self):
        ops = self.ops
        next_cluster = 0

        # 1. grow per-element clusters greedily
        for first in self.ops_sorted:
            first_node = ops.nodes[first]
            if first_node.cluster_id is not None or not first_node.op.is_per_element():
                continue
            element_count = first_node.shape.element_count()
            cid = next_cluster
            next_cluster += 1
            self.clusters[cid] = Cluster(kernel=None)
            first_node.cluster_id = cid

            grown = True
            while grown:
                grown = False
                for other in self.ops_sorted:
                    node = ops.nodes[other]
                    if (
                        node.cluster_id is not None
                        or not node.op.is_per_element()
                        or node.shape.element_count() != element_count
                    ):
                        continue
                    # every edge shared with the cluster must be a plain per-element edge
                    has_neighbor = False
                    blocked = False
                    for e in ops.in_edges(other):
                        edge = ops.edges[e]
                        if ops.nodes[edge.src].cluster_id == cid:
                            has_neighbor = True
                            if not edge.is_per_element(ops.nodes[edge.dst].op):
                                blocked = True
                                break
                    if not blocked:
                        for e in ops.out_edges(other):
                            edge = ops.edges[e]
                            if ops.nodes[edge.dst].cluster_id == cid:
                                has_neighbor = True
                                if not edge.is_per_element(ops.nodes[edge.dst].op):
                                    blocked = True
                                    break
                    if blocked or not has_neighbor:
                        continue

                    def outside_feeding_cluster(n):
                        return ops.nodes[n].cluster_id is None and any(
                            ops.nodes[s].cluster_id == cid for s in ops.successors(n)
                        )

                    def outside_fed_by_cluster(n):
                        return ops.nodes[n].cluster_id is None and any(
                            ops.nodes[p].cluster_id == cid for p in ops.predecessors(n)
                        )

                    # no path may leave the cluster and come back
                    if self._any_successor([other], outside_feeding_cluster):
                        continue
                    if self._any_predecessor([other], outside_fed_by_cluster):
                        continue
                    node.cluster_id = cid
                    grown = True
                    break

        # 2. turn each per-element cluster into a kernel
        for cid, cluster in self.clusters.items():
            members = [n for n in self.ops_sorted if ops.nodes[n].cluster_id == cid]
            element_count = ops.nodes[members[0]].shape.element_count()
            k_inputs: List[View] = []
            k_ops: List[object] = []
            k_outputs: List[int] = []
            arg_op_index: Dict[ArgSource, int] = {}
            member_op_index: Dict[int, int] = {}
            for nid in members:
                args = []
                for source in get_arg_sources(ops, nid):
                    if source.node_id in member_op_index:
                        args.append(member_op_index[source.node_id])
                        continue
                    if source not in arg_op_index:
                        src_node = ops.nodes[source.node_id]
                        if source.is_gather:
                            arg_op_index[source] = len(k_inputs)  # an input index, not an op index
                            k_inputs.append(source.view)
                            cluster.inputs.append(source.node_id)
                        else:
                            assert src_node.cluster_id != cid
                            arg_op_index[source] = len(k_ops)
                            if src_node.op.kind == "Literal":
                                k_ops.append(PeLiteral(src_node.op.a))
                            elif src_node.op.kind == "Coord":
                                k_ops.append(PeCoord(source.view))
                            elif src_node.op.kind == "Rand":
                                k_ops.append(PeRand(src_node.op.a, source.view))
                            else:
                                k_ops.append(PeLoad(len(k_inputs)))
                                k_inputs.append(source.view)
                                cluster.inputs.append(source.node_id)
                    args.append(arg_op_index[source])
                op = ops.nodes[nid].op
                if op.kind == "Unary":
                    k_ops.append(PeUnary(op.a, args[0]))
                elif op.kind == "Binary":
                    k_ops.append(PeBinary(op.a, (args[0], args[1])))
                elif op.kind == "Select":
                    k_ops.append(PeSelect(op.a, tuple(args[:4])))
                elif op.kind == "Gather":
                    k_ops.append(PeGather(ops.nodes[nid].shape, op.a, args[0], args[1]))
                else:
                    raise AssertionError(f"unexpected op {op} in per-element cluster")
                member_op_index[nid] = len(k_ops) - 1
                if any(ops.nodes[s].cluster_id != cid for s in ops.successors(nid)):
                    k_outputs.append(len(k_ops) - 1)
                    cluster.outputs.append(ClusterOutput(nid))
            cluster.kernel = PerElementKernel(element_count, tuple(k_inputs), tuple(k_outputs), tuple(k_ops))

        # 3. one cluster per remaining compute node
        for nid in self.ops_sorted:
            node = ops.nodes[nid]
            if node.cluster_id is not None:
                continue
            op = node.op
            src = get_arg_sources(ops, nid)
            cluster = None
            if op.kind == "Reduce":
                assert len(src) == 1
                cluster = Cluster(
                    ReduceKernel(node.shape, src[0].view, op.a, op.b), [src[0].node_id], [ClusterOutput(nid)]
                )
            elif op.kind == "MatMul":
                assert len(src) == 2
                cluster = Cluster(
                    MatMulKernel(node.shape, op.a, src[0].view, src[1].view),
                    [src[0].node_id, src[1].node_id],
                    [ClusterOutput(nid)],
                )
            elif op.kind == "Unpad":
                assert len(src) == 1
                cluster = Cluster(
                    UnpadKernel(node.shape, src[0].view, op.a, op.b), [src[0].node_id], [ClusterOutput(nid)]
                )
            elif op.kind == "WindowsToImage":
                assert len(src) == 1
                cluster = Cluster(
                    WindowsToImageKernel(node.shape, src[0].view, tuple(op.a)),
                    [src[0].node_id],
                    [ClusterOutput(nid)],
                )
            elif op.kind == "ScatterAdd":
                assert len(src) == 3
                acc, values, indices = src
                assert acc.view.is_contiguous() or ops.nodes[acc.node_id].op.kind == "Literal"
                cluster = Cluster(
                    ScatterAddKernel(node.shape, values.view, op.a, indices.view),
                    [values.node_id, indices.node_id],
                    [ClusterOutput(nid, copy_from=acc.node_id)],
                )
            elif op.kind in ("Input", "Output", "Literal", "Coord", "Rand"):
                continue
            else:
                raise AssertionError(f"per-element op {op} left unclustered")
            cid = next_cluster
            next_cluster += 1
            self.clusters[cid] = cluster
            node.cluster_id = cid

        # 4. order the clusters
        succ: Dict[int, List[int]] = {c: [] for c in self.clusters}
        pred: Dict[int, List[int]] = {c: [] for c in self.clusters}
        for eid in sorted(ops.edges):
            e = ops.edges[eid]
            a, b = ops.nodes[e.src].cluster_id, ops.nodes[e.dst].cluster_id
            if a is None or b is None or a == b:
                continue
            succ[a].append(b)
            pred[b].append(a)
        stack = [c for c in self.clusters if not pred[c]]
        done = set()
        self.clusters_sorted = []
        while stack:
            c = stack.pop()
            if c in done:
                continue
            done.add(c)
            self.clusters_sorted.append(c)
            for d in reversed(succ[c]):
                if d not in done and all(p in done for p in pred[d]):
                    stack.append(d)
        assert len(self.clusters_sorted) == len(self.clusters), "cluster graph has a cycle"

    # -- reporting -----------------------------------------------------------
    def kernel_labels(self) -> List[str]:
        return [self.clusters[c].kernel.label_name() for c in self.clusters_sorted]

    def fill_kernel_for(self, cluster_output: ClusterOutput) -> Optional[FillKernel]:
        """The Fill the executor must run first when a ScatterAdd accumulator
        starts from a literal (src/environment.rs:419-436)."""
        if cluster_output.copy_from is None:
            return None
        src = self.ops.nodes[cluster_output.copy_from]
        if src.op.kind != "Literal":
            return None
        return FillKernel(src.op.a, self.ops.nodes[cluster_output.node_id].shape.element_count())
