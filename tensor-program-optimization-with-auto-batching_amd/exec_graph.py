"""The auto-batching dataflow graph.

A request is a chain of operations (encode_prompt -> prefill -> decode -> decode_answer [-> print]) joined by
variables; every `generate()` of the front end appends one chain.  The graph is bipartite and is walked in
*frontiers*: the source variables, the operations that read them, the variables those write, and so on.  Because all
chains have the same shape, the decode operations of all requests meet on one frontier, and `fuse_batchable_ops`
folds them into a single operation that carries every request's input and output variable - the batched decode.

Same behaviour as `tvm/llama_auto_batcher/exec_graph.py:4-121` (VarNode / OpNode / ExecGraph, `ms_bfs`,
`fuse_batchable_ops`, `get_max_batch_sizes`), with two deliberate differences: frontiers are insertion-ordered
lists, not sets, so the order in which operations run does not depend on object hashes; and an unknown node type
raises instead of ending the process.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Iterable, Iterator, List


@dataclass(eq=False)
class VarNode:
    """A value flowing between operations; `ops` are its readers."""
    id: int
    var: Any
    ops: List["OpNode"] = field(default_factory=list)


@dataclass(eq=False)
class OpNode:
    """An operation; after fusion it may hold the variables and sequence ids of many requests, position by position."""
    op_type: str
    input_vars: List[VarNode] = field(default_factory=list)
    output_vars: List[VarNode] = field(default_factory=list)
    seqids: List[int] = field(default_factory=list)

    def absorb(self, other: "OpNode") -> None:
        """Take over another operation of the same type: its variables, its sequences, and its place among the
        readers of its inputs."""
        for v in other.input_vars:
            v.ops = [self if op is other else op for op in v.ops]
        self.input_vars.extend(other.input_vars)
        self.output_vars.extend(other.output_vars)
        self.seqids.extend(other.seqids)


Frontier = List[Any]


def _unique(nodes: Iterable[Any]) -> Frontier:
    """First occurrence of every node, by identity."""
    return list({id(n): n for n in nodes}.values())


def _successors(node: Any) -> List[Any]:
    if isinstance(node, VarNode):
        return node.ops
    if isinstance(node, OpNode):
        return node.output_vars
    raise TypeError(f"unknown node type {type(node)}")


class ExecGraph:
    def __init__(self, batchable_op_types: Iterable[str]):
        self.batchable_op_types = tuple(batchable_op_types)
        self.sources: List[VarNode] = []
        self.op_nodes: List[OpNode] = []
        self._n_vars = 0

    # ------------------------------------------------------------------ construction
    @property
    def var_id(self) -> int:
        """Id of the variable created last (-1 before the first)."""
        return self._n_vars - 1

    def add_source(self, var: VarNode) -> None:
        self.sources.append(var)

    def variable(self, var: Any, source: bool) -> VarNode:
        node = VarNode(self._n_vars, var)
        self._n_vars += 1
        if source:
            self.add_source(node)
        return node

    def operation(self, input_var: VarNode, op_type: str, seqid=None, output_var: VarNode = None) -> OpNode:
        op = OpNode(op_type, [input_var], [] if output_var is None else [output_var], [] if seqid is None else [seqid])
        input_var.ops.append(op)
        self.op_nodes.append(op)
        return op

    # ------------------------------------------------------------------ traversal
    def _frontiers(self, rewrite: Callable[[Frontier], Frontier] = None) -> Iterator[Frontier]:
        """The frontiers after the sources, in order.  `rewrite` may replace a frontier before the walk goes on
        from it (fusion does)."""
        frontier = _unique(self.sources)
        while frontier:
            frontier = _unique(s for node in frontier for s in _successors(node))
            if rewrite is not None:
                frontier = _unique(rewrite(frontier))
            if frontier:
                yield frontier

    def ms_bfs(self, f: Callable[[Frontier], Frontier] = lambda frontier: frontier) -> None:
        """Multi-source breadth-first walk: `f` sees every frontier after the sources and returns the frontier to
        continue from."""
        for _ in self._frontiers(f):
            pass

    def levels(self) -> List[Frontier]:
        return list(self._frontiers())

    @staticmethod
    def _is_op_frontier(frontier: Frontier) -> bool:
        return bool(frontier) and isinstance(frontier[0], OpNode)    # a frontier is all variables or all operations

    # ------------------------------------------------------------------ queries and passes
    def get_max_batch_sizes(self) -> dict:
        """Largest number of requests held by one operation, per batchable operation type."""
        sizes: dict = {}
        for op in self.op_nodes:
            if op.op_type in self.batchable_op_types:
                sizes[op.op_type] = max(len(op.input_vars), sizes.get(op.op_type, 0))
        return sizes

    def fuse_batchable_ops(self) -> None:
        """On every operation frontier, fold the batchable operations of one type into the first of them."""
        def fold(frontier: Frontier) -> Frontier:
            if not self._is_op_frontier(frontier):
                return frontier
            keeper: dict = {}
            kept: Frontier = []
            for op in frontier:
                first = keeper.setdefault(op.op_type, op) if op.op_type in self.batchable_op_types else op
                if first is op:
                    kept.append(op)
                else:
                    first.absorb(op)
                    self.op_nodes = [o for o in self.op_nodes if o is not op]
            return kept
        self.ms_bfs(fold)

    def print(self) -> None:
        for frontier in self._frontiers():
            if self._is_op_frontier(frontier):
                for op in frontier:
                    print(f"Op(type={op.op_type}, seqids={op.seqids}, in_ids={[v.id for v in op.input_vars]}, "
                          f"out_ids={[v.id for v in op.output_vars]})")
            else:
                print(" ".join(f"Var(id={v.id})" for v in frontier))

    # ------------------------------------------------------------------ execution
    def execute_op(self, op_node: OpNode) -> None:
        """Overridden by the model-specific graph."""

    def execute(self) -> None:
        for frontier in self._frontiers():
            if self._is_op_frontier(frontier):
                for op in frontier:
                    self.execute_op(op)
