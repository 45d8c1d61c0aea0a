"""Shared driver code: tensor recipes, module loading, the timing protocol.

Timing follows the reference's drivers (convert_eval_rms.py:253-275): ten
warm-up calls on a side stream, one `forward` captured in a graph, 100 replays
between events, mean per replay.
"""
import importlib.util
import json
import os
import sys

import torch

from ..codegen.convert_module import convert_ir_to_triton

HERE = os.path.dirname(os.path.abspath(__file__))
dtype = torch.float16


def load_config(name):
    with open(os.path.join(HERE, name)) as f:
        return json.load(f)


def generate_module(ir_code, constants, output_file):
    src = convert_ir_to_triton(ir_code, None, constants)
    os.makedirs(os.path.dirname(os.path.abspath(output_file)), exist_ok=True)
    with open(output_file, "w") as f:
        f.write(src)
    return src


def load_module(path, name):
    spec = importlib.util.spec_from_file_location(name, path)
    module = importlib.util.module_from_spec(spec)
    sys.modules[name] = module
    spec.loader.exec_module(module)
    return module


def positional_args(module, tensors, blocks):
    args = []
    for p in module.TENSOR_PARAMS:
        if p not in tensors:
            raise ValueError("Unknown tensor parameter: %s" % p)
        args.append(tensors[p])
    for p in module.BLOCK_PARAMS:
        if p not in blocks:
            raise ValueError("Unknown block parameter: %s" % p)
        args.append(blocks[p])
    return args


def time_graph_ms(fn, device, warmup=10, iters=100):
    stream = torch.cuda.Stream(device)
    with torch.cuda.stream(stream):
        for _ in range(warmup):
            fn()
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            fn()
    stream.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        start.record()
        for _ in range(iters):
            graph.replay()
        end.record()
    stream.synchronize()
    return start.elapsed_time(end) / iters


def time_eager_ms(fn, iters=20, warmup=3):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def attention_tensors(M, N, D, P, H, device, seed=42, std=0.01):
    """The tensor dictionary of the reference's drivers (convert_eval_rms.py:126-176, plus the names only the
    sweep drivers define, benchmark/keyformer_llama_benchmark.py:40-80: Q2/K2/V2, O1, C_div_perturb), i.e.
    every name a generated module can ask for."""
    torch.manual_seed(seed)
    if device.type == "cuda":
        torch.cuda.manual_seed(seed)
    r = lambda *s: torch.randn(s, device=device, dtype=dtype) * std
    z = lambda *s, dt=dtype: torch.zeros(s, device=device, dtype=dt)
    L = P + M
    return {
        "X": r(M, N), "X2": z(M), "X_norm": z(M, N),
        "WQ": r(N, N), "WK": r(N, N), "WV": r(N, N),
        "K_cache": r(H, L, D), "V_cache": r(H, L, D),
        "C": z(H, M, L), "C_exp": z(H, M, L, dt=torch.float32), "C_div": z(H, M, L, dt=torch.float32),
        "C_sum": z(H, M, dt=torch.float32),
        "Q": z(H, M, D), "K": z(H, M, D), "V": z(H, M, D), "Q1": z(M, N), "K1": z(M, N), "V1": z(M, N),
        "O": z(H, M, D), "O2": z(M, N),
        "noise": torch.randn((H, M, L), device=device, dtype=dtype),
        "C_perturb": z(H, M, L), "C_exp_perturb": z(H, M, L), "C_sum_perturb": z(H, M),
        "C_out": z(H, L), "C_out1": z(H, L), "C_out2": z(H, L),
        "Q_norm": z(H, M, D), "K_norm": z(H, M, D),
        "Q2": z(M, H, D), "K2": z(M, H, D), "V2": z(M, H, D), "O1": z(M, H, D), "C_div_perturb": z(H, M, L),
    }


def ffn_tensors(M, N, P, device, seed=42, scale=0.001):
    """The reference's FFN driver recipe (convert_ffn_llama.py:79-107)."""
    torch.manual_seed(seed)
    if device.type == "cuda":
        torch.cuda.manual_seed(seed)
    r = lambda *s: torch.randn(s, device=device, dtype=dtype).clamp(-1, 1) * scale
    z = lambda *s, dt=dtype: torch.zeros(s, device=device, dtype=dt)
    return {
        "O2": r(M, N), "X": r(M, N), "WO": r(N, N), "WFF1a": r(N, P), "WFF1b": r(N, P), "WFF2": r(P, N),
        "attn_O1": z(M, N), "attn_O2": z(M, N), "attn_O3": z(M), "attn_O_norm": z(M, N),
        "FF1a": z(M, P), "FF1b": z(M, P), "FF1b_silu": z(M, P), "FF1": z(M, P), "FF2": z(M, N),
        "O_FF": z(M, N), "O_FF1": z(M), "O_FF_norm": z(M, N),
    }
