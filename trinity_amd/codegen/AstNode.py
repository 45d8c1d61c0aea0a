"""AST node of the tile-level IR (reference: codegen/AstNode.py:5-13)."""
from dataclasses import dataclass, field
from typing import Any, List

from .NodeType import NodeType


@dataclass
class ASTNode:
    node_type: NodeType
    children: List["ASTNode"] = field(default_factory=list)
    value: Any = None

    def __repr__(self):
        if self.value is not None:
            return "%s(%s)" % (self.node_type.value, self.value)
        return "%s(%s)" % (self.node_type.value, self.children)

    def walk(self):
        """Pre-order traversal."""
        yield self
        for c in self.children:
            yield from c.walk()
