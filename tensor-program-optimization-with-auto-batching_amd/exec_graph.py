"""The auto-batching dataflow graph: variables, operations, level-synchronous traversal, fusion of
batchable operations.  Restates `tvm/llama_auto_batcher/exec_graph.py:4-121`.

Each `generate()` call of a request adds a chain encode_prompt -> prefill -> decode -> decode_answer;
`fuse_batchable_ops` merges the `decode` nodes that sit on the same BFS level into one node, so that all
requests decode in one batched loop.
"""
from __future__ import annotations


class VarNode:
    def __init__(self, id, var):
        self.id = id
        self.var = var
        self.ops = []


class OpNode:
    def __init__(self, op_type):
        self.op_type = op_type
        self.input_vars = []
        self.output_vars = []
        self.seqids = []


class ExecGraph:
    def __init__(self, batchable_op_types):
        self.sources = []
        self.op_nodes = []
        self.batchable_op_types = list(batchable_op_types)
        self.var_id = -1

    def add_source(self, var):
        self.sources.append(var)

    def variable(self, var, source):
        self.var_id += 1
        node = VarNode(self.var_id, var)
        if source:
            self.add_source(node)
        return node

    def operation(self, input_var, op_type, seqid=None, output_var=None):
        op = OpNode(op_type)
        input_var.ops.append(op)
        op.input_vars.append(input_var)
        if output_var is not None:
            op.output_vars.append(output_var)
        if seqid is not None:
            op.seqids.append(seqid)
        self.op_nodes.append(op)
        return op

    def get_max_batch_sizes(self):
        sizes = {}
        for op in self.op_nodes:
            if op.op_type in self.batchable_op_types:
                sizes[op.op_type] = max(sizes.get(op.op_type, 0), len(op.input_vars))
        return sizes

    def ms_bfs(self, f=lambda level: level):
        """Multi-source BFS by levels; a level is all variables or all operations.  `f` may replace the
        level (used by fusion).  Levels keep insertion order, so traversal is deterministic."""
        visit = _ordered(self.sources)
        while visit:
            nxt = []
            for node in visit:
                children = node.ops if isinstance(node, VarNode) else node.output_vars
                if not isinstance(node, (VarNode, OpNode)):
                    raise TypeError(f"unknown node type {type(node)}")
                nxt.extend(children)
            visit = _ordered(f(_ordered(nxt)))

    def levels(self):
        out = []
        self.ms_bfs(lambda level: (out.append(level), level)[1])
        return out

    def print(self):
        def show(level):
            for node in level:
                if isinstance(node, VarNode):
                    print(f"Var(id={node.id})", end=" ")
                else:
                    print(f"Op(type={node.op_type}, seqids={node.seqids}, in_ids={[v.id for v in node.input_vars]}, "
                          f"out_ids={[v.id for v in node.output_vars]})")
            if level and isinstance(level[0], VarNode):
                print("")
            return level
        self.ms_bfs(show)

    def fuse_batchable_ops(self):
        def fuse(level):
            if not level or isinstance(level[0], VarNode):
                return level
            merged = {}
            out = []
            for node in level:
                if node.op_type not in self.batchable_op_types:
                    out.append(node)
                elif node.op_type in merged:
                    tgt = merged[node.op_type]
                    tgt.input_vars += node.input_vars
                    tgt.output_vars += node.output_vars
                    tgt.seqids += node.seqids
                    for v in node.input_vars:
                        v.ops[v.ops.index(node)] = tgt
                    if node in self.op_nodes:
                        self.op_nodes.remove(node)
                else:
                    merged[node.op_type] = node
                    out.append(node)
            return out
        self.ms_bfs(fuse)

    def execute_op(self, op_node):
        pass

    def execute(self):
        def run(level):
            if level and isinstance(level[0], OpNode):
                for node in level:
                    self.execute_op(node)
            return level
        self.ms_bfs(run)


def _ordered(nodes):
    seen = set()
    out = []
    for n in nodes:
        if id(n) not in seen:
            seen.add(id(n))
            out.append(n)
    return out
