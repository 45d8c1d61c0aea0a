"""Front end: tile-level IR text -> generated module source (the reference's
codegen/ package surface: IRParser, ASTNode, NodeType, convert_ir_to_triton)."""
from .AstNode import ASTNode  # noqa: F401
from .IrParser import IRParser  # noqa: F401
from .NodeType import NodeType  # noqa: F401
from .convert_module import convert_ir_to_triton  # noqa: F401
