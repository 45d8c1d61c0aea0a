"""FFN entry points (reference: convert_ffn_llama.py / convert_ffn_falcon.py, flags --n --o)."""
import argparse
import os

import torch

from . import baselines, cases, harness


def run(model, argv=None):
    ap = argparse.ArgumentParser(description="Convert the FFN IR to a generated module and run it")
    ap.add_argument("--n", type=int, default=0, help="Case number to convert")
    ap.add_argument("--o", type=int, default=0, help="0 only convert, 1 only test, 2 both convert and test")
    ap.add_argument("--dir", type=str, default=os.path.join(os.getcwd(), "evaluation"))
    args = ap.parse_args(argv)
    cfg = harness.load_config("ffn_%s_tensor_configs.json" % model)[0]
    M, N = cfg["M"], cfg["N"]
    falcon = model == "falcon"
    P = N if falcon else cfg["P"]   # the reference's Falcon FFN uses N x N weights (convert_ffn_falcon.py)
    sub = os.path.join(args.dir, "ffn", "ffn_%s" % model)
    case_file = os.path.join(sub, "ffn_%s_case%d.txt" % (model, args.n))
    output_file = os.path.join(sub, "ffn_%s_benchmark%d.py" % (model, args.n))
    if args.o in (0, 2):
        ir = open(case_file).read().strip() if os.path.exists(case_file) else cases.ffn_ir(N, P, falcon_tail=falcon)
        harness.generate_module(ir, {"M": M, "N": N, "P": P}, output_file)
        print("module written to", output_file)
    if args.o == 0:
        return 0
    if not torch.cuda.is_available():
        raise SystemExit("running the generated module needs a GPU (there is no CPU fallback)")
    device = torch.device("cuda:0")
    t = harness.ffn_tensors(M, N, P, device)
    module = harness.load_module(output_file, "ffn_%s_best" % model)
    # block parameters are deliberately not passed (convert_ffn_llama.py:166-170)
    tensor_args = [t[p] for p in module.TENSOR_PARAMS]
    ms = harness.time_graph_ms(lambda: module.forward(*tensor_args), device)
    print("Kernel execution completed!: %f ms" % ms)
    eager = baselines.SimpleFFN(M, N, P, t["WO"], t["WFF1a"], t["WFF1b"], t["WFF2"], falcon_tail=falcon)
    with torch.no_grad():
        want = eager(t["O2"], t["X"])
        base_ms = harness.time_eager_ms(lambda: eager(t["O2"], t["X"]))
    got = t["O_FF_norm"] if falcon else t["FF2"]
    print("PyTorch eager: %f ms" % base_ms)
    tol = dict(rtol=1e-2, atol=1e-2) if falcon else dict(rtol=1e-3, atol=1e-4)   # convert_ffn_llama.py:224
    ok = torch.allclose(got, want, **tol)
    print("all close to eager:", ok)
    return 0 if ok else 1
