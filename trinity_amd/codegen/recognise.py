"""Classify a parsed IR as one of the evaluated computations and extract the
numbers the hand-written kernels need.

The reference lowers *any* expression tree to Triton (codegen/TritonGen.py);
its evaluated computations are nine families only (README.md:25-30).  This
front end recognises those families by their tensor fingerprint and refuses
everything else instead of guessing.
"""
from dataclasses import dataclass, field
from typing import Dict, Optional

from .analysis import IRInfo


class UnsupportedIR(NotImplementedError):
    pass


@dataclass
class Computation:
    family: str                        # attention | ffn | rmsnorm
    variant: str = "vanilla"           # attention: vanilla | keyformer | roco
    prenorm: bool = False
    qknorm: bool = False
    falcon_tail: bool = False          # ffn: trailing residual + RMSNorm (output O_FF_norm)
    dims: Dict[str, int] = field(default_factory=dict)   # M, N, D, H, P (attention) / M, N, P (ffn)
    tau: float = 1.5


_ATTN_IN = {"X", "WQ", "WK", "WV"}
_FFN_IN = {"O2", "WO", "X", "WFF1a", "WFF1b", "WFF2"}


def _loop(info: IRInfo, var: str, kind: Optional[str] = None):
    for l in info.loops:
        if l.var == var and (kind is None or l.kind == kind):
            return l
    return None


def recognise(info: IRInfo, constants: Optional[Dict[str, int]] = None) -> Computation:
    constants = dict(constants or {})
    inputs, outputs = set(info.names("input")), set(info.names("output"))
    tensors = set(info.names("tensor"))

    if _ATTN_IN <= inputs and "O2" in outputs:
        c = Computation("attention")
        if "C_out" in outputs or "noise" in inputs:
            c.variant = "keyformer"
        elif {"C_out1", "C_out2"} <= outputs:
            c.variant = "roco"
        c.qknorm = bool({"Q_norm", "K_norm"} & tensors)
        c.prenorm = bool({"X2", "X_norm"} & (tensors | inputs)) and "sqr" in info.ops
        k_loop, p_loop = _loop(info, "k", "sloop"), _loop(info, "p", "sloop")
        # multi-kernel splits run the projection under its own ploop over n with a symbolic tile; the head
        # loop is the ploop over n whose tile is the head dimension
        n_loops = [l for l in info.loops if l.var == "n" and l.kind == "ploop"]
        n_loop = next((l for l in n_loops if isinstance(l.tile, int)), n_loops[0] if n_loops else None)
        if n_loop is None or k_loop is None:
            raise UnsupportedIR("attention IR without the head ploop / projection sloop")
        if not isinstance(n_loop.tile, int):
            raise UnsupportedIR("the head ploop must have a numeric tile (= head_dim)")
        d = {"N": int(n_loop.end), "D": int(n_loop.tile)}
        d["H"] = d["N"] // d["D"]
        if info.const_tiles:
            d["P"], d["M"] = int(info.const_tiles[0][0]), int(info.const_tiles[0][1])
        elif p_loop is not None:
            d["P"], d["M"] = 0, int(p_loop.end)
        else:
            d["P"] = 0
        for k in ("M", "N", "D", "H", "P"):
            if k in constants:
                d[k] = int(constants[k])
        if "M" not in d:
            raise UnsupportedIR("cannot determine the token count M")
        c.dims = d
        for lit in info.literals:
            if "." in lit:
                c.tau = float(lit)
        return c

    if _FFN_IN <= inputs and ({"FF2", "O_FF_norm"} & outputs):
        c = Computation("ffn")
        c.falcon_tail = "O_FF_norm" in outputs
        n_loop = _loop(info, "n", "ploop")
        p_loop = _loop(info, "p")
        d = {}
        if n_loop is not None:
            d["N"] = int(n_loop.end)
        d["P"] = int(p_loop.end) if p_loop is not None else d.get("N", 0)
        for k in ("M", "N", "P"):
            if k in constants:
                d[k] = int(constants[k])
        c.dims = d
        return c

    if inputs == {"O_FF"} and "O_FF_norm" in outputs:
        return Computation("rmsnorm", dims={k: int(v) for k, v in constants.items() if k in ("M", "N")})

    raise UnsupportedIR(
        "IR is not one of the evaluated computations (attention variants, FFN block, RMSNorm): inputs %s outputs %s"
        % (sorted(inputs), sorted(outputs))
    )
