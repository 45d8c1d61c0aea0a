"""Sweep driver: time every expression of an IR list, as the reference's
benchmark/*_benchmark.py drivers do (input format `<id>: <expression>` per
line, vanilla_llama_benchmark.py:141-161; one result record per expression with
the fields `ir_id`, `ir_expression`, `execution_time_ms`, `tensor_config`,
`error`, :388-401; flags --ir --output --start --num --end --topk, :746-753;
output tensors zeroed before every candidate, :237-240; NaN check on the result
after the timed replays, :288-291 - a printed warning, as there; the result
records keep the reference's five fields).

Every expression of one computation converts to a module over the same HIP
kernels, so the sweep measures that the whole list is accepted and how long the
call takes, not differences between the search's candidates.

    python -m trinity_amd.evaluation.sweep --ir cases.txt --m llama --output results.json
"""
import argparse
import json
import math
import os
import sys
import types

import torch

from ..codegen.analysis import analyse
from ..codegen.convert_module import convert_ir_to_triton
from ..codegen.IrParser import IRParser
from ..codegen.recognise import recognise
from . import harness


def parse_ir_file(path):
    """[(ir_id, expression)] from `<id>: <expression>` lines, or from a result JSON of an earlier sweep."""
    if path.endswith(".json"):
        with open(path) as f:
            return [(int(e["ir_id"]), e["ir_expression"]) for e in json.load(f) if isinstance(e, dict) and e.get("ir_expression")]
    out = []
    with open(path) as f:
        for line in f:
            line = line.strip()
            if not line or ":" not in line:
                continue
            head, expr = line.split(":", 1)
            try:
                ir_id = int(head)
            except ValueError:
                continue
            if "dummydata" not in expr:
                out.append((ir_id, expr.strip()))
    return out


def select(expressions, start=None, num=None, to_end=False):
    if start is not None:
        expressions = [(i, e) for i, e in expressions if i >= start]
        if num and not to_end:
            expressions = expressions[:num]
    return expressions


def tensor_config(ir, model):
    """The constants of the model's tensor-metadata config that apply to this expression's family."""
    family = recognise(analyse(IRParser().parse(ir)), None).family
    if family == "attention":
        return family, dict(harness.load_config("%s_configs.json" % model)[0])
    if family == "ffn":
        cfg = harness.load_config("ffn_%s_tensor_configs.json" % model)[0]
        P = cfg["N"] if model == "falcon" else cfg["P"]   # the reference's Falcon FFN uses N x N weights
        return family, {"M": cfg["M"], "N": cfg["N"], "P": P}
    raise ValueError("the sweep covers the attention variants and the FFN block")


# the tensors the reference's drivers clear before each candidate (vanilla_llama_benchmark.py:237-240, plus the
# score outputs of the KeyFormer / RoCo drivers and the FFN block's outputs)
_ATTN_OUTPUTS = ("O2", "Q1", "K1", "V1", "Q2", "K2", "V2", "Q", "K", "V", "C", "C_exp", "C_sum", "C_div", "O", "O1",
                 "X2", "X_norm", "C_out", "C_out1", "C_out2")
_FFN_OUTPUTS = ("attn_O1", "attn_O2", "attn_O3", "attn_O_norm", "FF1a", "FF1b", "FF1b_silu", "FF1", "FF2", "O_FF",
                "O_FF1", "O_FF_norm")


def run_one(ir_id, ir, model, device, convert_only=False):
    rec = {"ir_id": ir_id, "ir_expression": ir, "execution_time_ms": math.inf, "tensor_config": None, "error": None,
           "has_nan": None}
    try:
        family, cfg = tensor_config(ir, model)
        rec["tensor_config"] = cfg
        src = convert_ir_to_triton(ir, None, cfg)
        if convert_only:
            rec["error"] = "converted, not run"
            return rec
        module = types.ModuleType("%s_kernel_%d" % (model, ir_id))
        exec(compile(src, "<generated %d>" % ir_id, "exec"), module.__dict__)
        if family == "attention":
            t = harness.attention_tensors(cfg["M"], cfg["N"], cfg["D"], cfg["P"], cfg["H"], device)
            outputs, result = _ATTN_OUTPUTS, "O2"
            args = harness.positional_args(module, t, {"block_k": 32, "block_p": 16, "block_n": 64})
        else:
            t = harness.ffn_tensors(cfg["M"], cfg["N"], cfg["P"], device)
            outputs, result = _FFN_OUTPUTS, ("O_FF_norm" if "O_FF_norm" in module.TENSOR_PARAMS else "FF2")
            args = [t[p] for p in module.TENSOR_PARAMS]
        for name in outputs:        # every candidate starts from zeroed outputs and intermediates
            if name in t:
                t[name].zero_()
        rec["execution_time_ms"] = harness.time_graph_ms(lambda: module.forward(*args), device)
        rec["has_nan"] = bool(torch.isnan(t[result]).any().item())
        if rec["has_nan"]:
            print("WARNING: NaN values detected in [%d] %s tensor!" % (ir_id, result))
    except Exception as e:  # a failed candidate is a record, not the end of the sweep
        rec["error"] = "%s: %s" % (type(e).__name__, e)
    return rec


def main(argv=None):
    ap = argparse.ArgumentParser(description="Time every expression of an IR list")
    ap.add_argument("--ir", required=True, help="IR list (`<id>: <expression>` lines) or a result JSON")
    ap.add_argument("--output", default="benchmark_results.json")
    ap.add_argument("--m", default="llama", help="model: llama or falcon")
    ap.add_argument("--start", type=int, default=None, help="first ir_id to run")
    ap.add_argument("--num", type=int, default=None, help="number of expressions from --start")
    ap.add_argument("--end", action="store_true", help="run from --start to the last expression")
    ap.add_argument("--topk", type=int, default=10)
    ap.add_argument("--convert-only", action="store_true", help="convert every expression, run nothing (no GPU needed)")
    args = ap.parse_args(argv)
    expressions = select(parse_ir_file(args.ir), args.start, args.num, args.end)
    print("Found %d IR expressions to benchmark" % len(expressions))
    if not args.convert_only and not torch.cuda.is_available():
        raise SystemExit("running the generated modules needs a GPU (there is no CPU fallback)")
    device = torch.device("cuda:0") if not args.convert_only else None
    results = [run_one(i, e, args.m, device, args.convert_only) for i, e in expressions]
    os.makedirs(os.path.dirname(os.path.abspath(args.output)), exist_ok=True)
    with open(args.output, "w") as f:
        json.dump([{k: (None if k == "execution_time_ms" and math.isinf(v) else v) for k, v in r.items() if k != "has_nan"}
                   for r in results], f, indent=2)
    good = sorted((r for r in results if r["error"] is None), key=lambda r: r["execution_time_ms"])
    print("%d valid, %d failed; results in %s" % (len(good), len(results) - len(good), args.output))
    for r in good[: args.topk]:
        print("  ir %d: %.5f ms" % (r["ir_id"], r["execution_time_ms"]))
    failed = [r for r in results if r["error"] is not None and not args.convert_only]
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main())
