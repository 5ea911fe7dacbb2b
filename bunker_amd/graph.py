"""Declarative one-token decode graph: tensors with roles, nodes with ordered inputs/outputs.

Counterpart of the ``Graph`` class of the reference (src/fusion.ts:47-184): same methods
(``input``, ``node``, ``t``, ``out``, ``externals``, ``deps``), same naming of produced tensors
(``n<id>_<output name>``).  The fusion explorer that lives in the same reference file is not
reproduced: here a node is served by a pre-compiled kernel and the only partitions are "every
node its own kernel" and the fixed hand-fused groups of ``runner.choosePartition``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


@dataclass
class TensorType:
    shape: list
    dtype: str            # "bf16" | "f32" | "i32" | "q4_k"
    strides: list = field(default_factory=list)


def row_major(shape, dtype) -> TensorType:
    strides = []
    for i in range(len(shape)):
        s = 1
        for d in shape[i + 1:]:
            s *= d
        strides.append(s)
    return TensorType(list(shape), dtype, strides)


@dataclass
class NodeIO:
    name: str
    tensorName: str
    type: TensorType
    role: str


@dataclass
class GraphNode:
    id: int
    op: str
    inputs: list
    outputs: list
    grid: list
    params: dict


@dataclass
class Tensor:
    name: str
    type: TensorType
    role: str             # "data" | "weight" | "state" | "scalar"
    producer: Any = None
    consumers: list = field(default_factory=list)


class Graph:
    def __init__(self):
        self.nodes: list[GraphNode] = []
        self.tensors: dict[str, Tensor] = {}
        self._next = 0

    def input(self, name: str, type: TensorType, role: str = "data") -> Tensor:
        t = Tensor(name, type, role)
        self.tensors[name] = t
        return t

    def node(self, op: str, inputs: list, outputs: list, grid, params: dict | None = None) -> GraphNode:
        """inputs: [(tensor | tensor name, arg name)], outputs: [(name, TensorType[, role])]."""
        nid = self._next
        self._next += 1
        n = GraphNode(nid, op, [], [], list(grid), dict(params or {}))
        for tensor, argname in inputs:
            t = self.tensors[tensor] if isinstance(tensor, str) else tensor
            n.inputs.append(NodeIO(argname, t.name, t.type, t.role))
            t.consumers.append(n)
        for o in outputs:
            oname, otype = o[0], o[1]
            role = o[2] if len(o) > 2 else "data"
            full = f"n{nid}_{oname}"
            n.outputs.append(NodeIO(oname, full, otype, role))
            self.tensors[full] = Tensor(full, otype, role, producer=n)
        self.nodes.append(n)
        return n

    def t(self, name: str) -> Tensor:
        if name not in self.tensors:
            raise KeyError(f'tensor "{name}" not found')
        return self.tensors[name]

    def out(self, node: GraphNode, output_name: str = "out") -> str:
        return f"n{node.id}_{output_name}"

    def externals(self) -> list[str]:
        return [t.name for t in self.tensors.values() if t.producer is None]

    def deps(self) -> dict[int, set]:
        m = {n.id: set() for n in self.nodes}
        for n in self.nodes:
            for i in n.inputs:
                p = self.tensors[i.tensorName].producer
                if p is not None:
                    m[n.id].add(p.id)
        return m
