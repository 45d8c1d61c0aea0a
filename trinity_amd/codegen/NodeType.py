"""Node kinds of the tile-level IR (same vocabulary as the reference's
codegen/NodeType.py:3-35, so IR text written for it parses here)."""
from enum import Enum


class NodeType(Enum):
    LOOP = "loop"
    PLOOP = "ploop"          # parallel loop: one workgroup per tile
    SLOOP = "sloop"          # sequential loop inside a workgroup
    INPUT = "input"
    OUTPUT = "output"
    TENSOR = "tensor"        # intermediate tensor
    TILE = "tile"
    FULLTILE = "fulltile"
    CONST_TILE = "const_tile"
    ELEM = "elem"
    INDEX = "index"
    LOAD = "load"
    STORE = "store"
    SEQ = "seq"
    DUMMY = "dummy"
    ADD = "+"
    SUB = "-"
    MUL = "x"                # element-wise product
    DIV = "/"
    MATMUL = "*"
    EXP = "exp"
    SQR = "sqr"
    SQRT = "sqrt"
    SIGMOID = "sigmoid"
    RSUM = "rsum"
    BCAST = "bcast"
    CONCAT = "concat"
    TRANSPOSE = "transpose"
    PERMUTE3 = "permute3"
    SQUEEZE = "squeeze"
    UNSQUEEZE = "unsqueeze"
    NUM = "num"
    VAR = "var"
