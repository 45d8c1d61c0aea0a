"""S-expression parser for the tile-level IR.

Grammar (as accepted by the reference's codegen/IrParser.py:13-130): lists
`(op child ...)`, `;` comments, integers, bare words (variables; `fulltile`
and `dummy` are nodes of their own), and the multi-name form
`(tensor Q1,K1,V1)` / `(input ...)` / `(output ...)` whose comma-separated
names become one VAR child each.
"""
import re
from typing import List

from .AstNode import ASTNode
from .NodeType import NodeType

_OPS = {t.value: t for t in NodeType if t not in (NodeType.NUM, NodeType.VAR, NodeType.LOOP)}
_NAMED = ("tensor", "input", "output")
_TOKEN = re.compile(r"\(|\)|,|[^\s(),]+")


class IRParser:
    def __init__(self):
        self.tokens: List[str] = []
        self.pos = 0

    def tokenize(self, code: str) -> List[str]:
        return _TOKEN.findall(re.sub(r";[^\n]*", "", code))

    def parse(self, code: str) -> ASTNode:
        self.tokens = self.tokenize(code)
        self.pos = 0
        if not self.tokens:
            raise ValueError("empty IR")
        node = self._expr()
        if self.pos != len(self.tokens):
            raise ValueError("trailing tokens after the root expression: %r" % self.tokens[self.pos:self.pos + 3])
        return node

    # -- internals
    def _peek(self):
        if self.pos >= len(self.tokens):
            raise ValueError("unexpected end of input")
        return self.tokens[self.pos]

    def _expr(self) -> ASTNode:
        tok = self._peek()
        if tok == "(":
            return self._list()
        if tok in (")", ","):
            raise ValueError("unexpected %r" % tok)
        self.pos += 1
        if re.fullmatch(r"-?\d+", tok):
            return ASTNode(NodeType.NUM, [], int(tok))
        if tok == "fulltile":
            return ASTNode(NodeType.FULLTILE, [])
        if tok == "dummy":
            return ASTNode(NodeType.DUMMY, [])
        return ASTNode(NodeType.VAR, [], tok)

    def _list(self) -> ASTNode:
        self.pos += 1  # "("
        op = self._peek()
        self.pos += 1
        if op not in _OPS:
            raise ValueError("Unknown operation: %s" % op)
        children = []
        if op in _NAMED:
            while self._peek() != ")":
                tok = self._peek()
                self.pos += 1
                if tok == ",":
                    continue
                if tok == "(":
                    raise ValueError("tensor names must be bare words")
                children.append(ASTNode(NodeType.VAR, [], tok))
            if not children:
                raise ValueError("(%s) needs at least one name" % op)
        else:
            while self._peek() != ")":
                children.append(self._expr())
        self.pos += 1  # ")"
        return ASTNode(_OPS[op], children)
