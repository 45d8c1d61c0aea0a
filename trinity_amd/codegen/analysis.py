"""Structural analysis of a parsed tile-level IR: kernels, loops, tensor roles
and the two metadata lists of the generated-module protocol.

The reference derives the same facts inside its Triton emitter
(codegen/TritonGen.py:349-425 kernels per top-level `seq` child, :563-573
TENSOR_PARAMS / BLOCK_PARAMS, :1018-1053 cross-kernel tensors, :1704-1883
tensors that must live in memory).  Here they only decide which buffers the
caller must pass; no code is emitted from the expression tree.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Set, Tuple

from .AstNode import ASTNode
from .NodeType import NodeType

_LOOPS = (NodeType.PLOOP, NodeType.SLOOP)
_NAMED = (NodeType.INPUT, NodeType.OUTPUT, NodeType.TENSOR)


@dataclass
class Loop:
    kind: str                 # "ploop" | "sloop"
    start: int
    end: int
    tile: object              # int (fixed tile) or str (symbolic tile -> block parameter)
    var: str
    kernel: int

    @property
    def block_param(self) -> Optional[str]:
        return None if isinstance(self.tile, int) else "block_" + self.var


@dataclass
class Access:
    name: str
    kind: str                 # "load" | "store"
    pattern: Tuple[str, ...]  # one entry per index item
    kernel: int
    loops: Tuple[int, ...]    # ids of the enclosing loop instances, outermost first
    sloop_vars: Tuple[str, ...]  # variables of the enclosing sloops


@dataclass
class IRInfo:
    kernels: List[ASTNode]
    loops: List[Loop]
    accesses: List[Access]
    roles: Dict[str, str]                      # tensor name -> input | output | tensor
    ops: Set[str]
    literals: Set[str]                         # non-integer literals (e.g. "1.5") and integer divisors
    const_tiles: List[Tuple[int, int]]
    tensor_params: List[str] = field(default_factory=list)
    block_params: List[str] = field(default_factory=list)

    def names(self, role):
        return sorted(n for n, r in self.roles.items() if r == role)


def _only_dummy(node: ASTNode) -> bool:
    if node.node_type == NodeType.DUMMY:
        return True
    if node.node_type == NodeType.SEQ:
        return all(_only_dummy(c) for c in node.children)
    if node.node_type in _LOOPS:
        return len(node.children) > 4 and _only_dummy(node.children[4])
    return False


def flatten_seq(node: ASTNode) -> List[ASTNode]:
    """Top-level `seq` children = kernels (dummy-only entries dropped)."""
    if node.node_type == NodeType.SEQ:
        out = []
        for c in node.children:
            out.extend(flatten_seq(c))
        return out
    if _only_dummy(node):
        return []
    return [node]


def _loop_field(n: ASTNode):
    if n.node_type == NodeType.NUM:
        return n.value
    return n.value if n.value is not None else repr(n)


def _index_pattern(index: ASTNode) -> Tuple[str, ...]:
    items = index.children if index.node_type == NodeType.INDEX else [index]
    pat = []
    for it in items:
        if it.node_type == NodeType.FULLTILE:
            pat.append("fulltile")
        elif it.node_type in (NodeType.TILE, NodeType.ELEM):
            v = it.children[0] if it.children else None
            pat.append("%s_%s" % (it.node_type.value, v.value if v is not None else ""))
        elif it.node_type == NodeType.CONST_TILE:
            pat.append("const_%s_%s" % tuple(c.value for c in it.children[:2]))
        else:
            pat.append(it.node_type.value)
    return tuple(pat)


def analyse(root: ASTNode) -> IRInfo:
    kernels = flatten_seq(root) if root.node_type == NodeType.SEQ else [root]
    loops: List[Loop] = []
    accesses: List[Access] = []
    roles: Dict[str, str] = {}
    ops: Set[str] = set()
    literals: Set[str] = set()
    const_tiles: List[Tuple[int, int]] = []
    loop_ids = [0]

    def visit(node: ASTNode, kid: int, stack: Tuple[int, ...], svars: Tuple[str, ...]):
        t = node.node_type
        ops.add(t.value)
        if t in _LOOPS:
            start, end, tile, var = (_loop_field(c) for c in node.children[:4])
            loop_ids[0] += 1
            loops.append(Loop(t.value, start, end, tile, var, kid))
            nstack = stack + (loop_ids[0],)
            nsv = svars + ((var,) if t == NodeType.SLOOP else ())
            for c in node.children[4:]:
                visit(c, kid, nstack, nsv)
            return
        if t in (NodeType.LOAD, NodeType.STORE):
            target = node.children[0]
            index = node.children[2] if t == NodeType.STORE else (node.children[1] if len(node.children) > 1 else None)
            if target.node_type in _NAMED:
                for nm in target.children:
                    role = target.node_type.value
                    prev = roles.get(nm.value)
                    if prev is None or role == "input" or (role == "output" and prev == "tensor"):
                        roles[nm.value] = role
                    if index is not None:
                        accesses.append(Access(nm.value, t.value, _index_pattern(index), kid, stack, svars))
            if t == NodeType.STORE:
                visit(node.children[1], kid, stack, svars)
            if index is not None:
                for it in index.walk():
                    if it.node_type == NodeType.CONST_TILE:
                        const_tiles.append(tuple(c.value for c in it.children[:2]))
            return
        if t == NodeType.VAR and node.value is not None and not str(node.value).isidentifier():
            literals.add(str(node.value))
        if t == NodeType.DIV and len(node.children) == 2 and node.children[1].node_type == NodeType.NUM:
            literals.add(str(node.children[1].value))
        for c in node.children:
            visit(c, kid, stack, svars)

    for kid, k in enumerate(kernels):
        visit(k, kid, (), ())

    info = IRInfo(kernels, loops, accesses, roles, ops, literals, const_tiles)
    info.block_params = sorted({l.block_param for l in loops if l.block_param})
    info.tensor_params = _tensor_params(info)
    return info


def _tensor_params(info: IRInfo) -> List[str]:
    """Buffers the caller passes: every input and output, plus each
    intermediate that cannot stay in registers - written in one kernel and
    read in another, accessed through more than one index pattern, or written
    inside one sequential loop and read inside a different one through an
    index that depends on that loop's variable."""
    keep = []
    by_name: Dict[str, List[Access]] = {}
    for a in info.accesses:
        by_name.setdefault(a.name, []).append(a)
    for name in sorted(info.roles):
        if info.roles[name] != "tensor":
            keep.append(name)
            continue
        acc = by_name.get(name, [])
        stores = [a for a in acc if a.kind == "store"]
        loads = [a for a in acc if a.kind == "load"]
        cross_kernel = any(s.kernel != l.kernel for s in stores for l in loads)
        patterns = {a.pattern for a in acc}
        cross_sloop = False
        for s in stores:
            for l in loads:
                if s.kernel != l.kernel or not s.sloop_vars or not l.sloop_vars:
                    continue
                uses_var = any(p == "tile_" + v or p == "elem_" + v for p in s.pattern for v in s.sloop_vars)
                if uses_var and s.loops != l.loops and (not s.loops or not l.loops or s.loops[-1] != l.loops[-1]):
                    cross_sloop = True
        if cross_kernel or len(patterns) > 1 or cross_sloop:
            keep.append(name)
    return keep
