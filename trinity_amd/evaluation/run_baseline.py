"""Baseline entry point, same flags as the reference's run_baseline.py:6-10
(--m model, --t variant, --b baseline, --pre).

The reference times competitor stacks there (TensorRT, FlashInfer, TorchInductor);
those are other projects' code and are not part of this build.  What remains
meaningful on an MI355X is the PyTorch-eager graph of the same computation
(`--b eager`, the reference's eager classes as restated in baselines.py), timed
with the same protocol next to this library's call (`--b trinity`).

    python -m trinity_amd.evaluation.run_baseline --t roco --m falcon --b eager
"""
import argparse

import torch

from . import baselines, cases, harness

NOT_BUILT = ("trt", "flashinfer", "inductor")


def main(argv=None):
    ap = argparse.ArgumentParser(description="Time a baseline of one evaluated computation")
    ap.add_argument("--m", type=str, default="llama", help="Input model type")
    ap.add_argument("--t", type=str, default="vanilla", help="RMS Type")
    ap.add_argument("--b", type=str, default="eager", help="Baseline Type: eager | trinity")
    ap.add_argument("--pre", action="store_true", help="Whether to use prenorm or not")
    args = ap.parse_args(argv)
    if args.b in NOT_BUILT:
        raise SystemExit("baseline %r is a third-party stack (TensorRT / FlashInfer / TorchInductor) and is not "
                         "part of this build; use --b eager or --b trinity" % args.b)
    if args.b not in ("eager", "trinity"):
        raise SystemExit("unknown baseline %r" % args.b)
    if not torch.cuda.is_available():
        raise SystemExit("timing needs a GPU")
    cfg = harness.load_config("%s_configs.json" % args.m)[0]
    M, D, N, P, H = (cfg[k] for k in ("M", "D", "N", "P", "H"))
    variant = args.t if args.t in ("keyformer", "roco") else "vanilla"
    prenorm = args.pre or args.t == "prenorm"
    qknorm = args.t == "qknorm"
    device = torch.device("cuda:0")
    t = harness.attention_tensors(M, N, D, P, H, device)
    if args.b == "eager":
        name = {("vanilla", False, False): "Vanilla", ("vanilla", True, False): "PreNorm", ("vanilla", False, True): "QKNorm",
                ("vanilla", True, True): "NormQKNorm", ("keyformer", False, False): "KeyFormer",
                ("keyformer", True, False): "NormKeyFormer", ("roco", False, False): "RoCo",
                ("roco", True, False): "NormRoCo"}.get((variant, prenorm, qknorm))
        if name is None:
            raise SystemExit("no eager baseline for this combination")
        kw = dict(W_q=t["WQ"], W_k=t["WK"], W_v=t["WV"])
        cls = getattr(baselines, name)
        model = (cls(M, N, D, P, t["noise"], t["K_cache"], t["V_cache"], **kw) if variant == "keyformer"
                 else cls(M, N, D, P, t["K_cache"], t["V_cache"], **kw))
        with torch.no_grad():
            ms = harness.time_graph_ms(lambda: model(t["X"]), device)
        print("PyTorch eager (%s, %s): %f ms" % (name, args.m, ms))
    else:
        import types

        from ..codegen.convert_module import convert_ir_to_triton

        src = convert_ir_to_triton(cases.attention_ir(variant, M, N, D, P, prenorm=prenorm, qknorm=qknorm), None, cfg)
        module = types.ModuleType("run_baseline_case")
        exec(compile(src, "<generated>", "exec"), module.__dict__)
        call_args = harness.positional_args(module, t, {"block_k": 32, "block_p": 16, "block_n": 64})
        ms = harness.time_graph_ms(lambda: module.forward(*call_args), device)
        print("trinity_amd (%s%s, %s): %f ms" % (args.t, " + prenorm" if args.pre else "", args.m, ms))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
