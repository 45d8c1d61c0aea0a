"""`convert_ir_to_triton`: same name and signature as the reference's entry
point (codegen/convert_module.py:5-13), same contract (IR text in, module
source text out) - but the returned module dispatches to the HIP library
instead of containing Triton kernels."""
from typing import Dict, Optional, Tuple

from .IrParser import IRParser
from .analysis import analyse
from .emit import emit_module
from .recognise import recognise


def convert_ir_to_triton(ir_code: str, tensor_shapes: Optional[Dict[str, Tuple]] = None,
                         constants: Optional[Dict[str, int]] = None) -> str:
    """Convert IR code to the source of a module exposing TENSOR_PARAMS,
    BLOCK_PARAMS and forward(...).  `tensor_shapes` is accepted for interface
    compatibility (shapes are taken from the tensors at call time)."""
    ast = IRParser().parse(ir_code)
    info = analyse(ast)
    comp = recognise(info, constants)
    return emit_module(info, comp)
