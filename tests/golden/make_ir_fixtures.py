"""Build tests/golden/ir_module_params.json from the reference's data files.

For every generated module the reference checks in under evaluation/ whose IR
survives in a result JSON of the same family (matched by ir_id, kernel count
and tensor names), record the IR text together with the TENSOR_PARAMS /
BLOCK_PARAMS lists the reference's generator wrote into that module.  Only
data is read (JSON fields and two list literals); nothing of the reference is
imported or executed.

    python tests/golden/make_ir_fixtures.py /root/reference
"""
import ast
import glob
import json
import os
import re
import sys


def main(ref):
    ev = os.path.join(ref, "evaluation")
    out = []
    for py in sorted(glob.glob(os.path.join(ev, "*", "*benchmark*.py")) + glob.glob(os.path.join(ev, "ffn", "*", "*benchmark*.py"))):
        src = open(py).read()
        mt = re.search(r"^TENSOR_PARAMS = (\[.*\])$", src, re.M)
        mb = re.search(r"^BLOCK_PARAMS = (\[.*\])$", src, re.M)
        num = re.search(r"benchmark_?(\d+)\.py$", py)
        if not (mt and mb and num):
            continue
        tparams, bparams, ir_id = ast.literal_eval(mt.group(1)), ast.literal_eval(mb.group(1)), int(num.group(1))
        n_kernels = len(re.findall(r"^def kernel_\d+", src, re.M))
        fam, base = os.path.dirname(py), os.path.basename(py)
        for js in sorted(glob.glob(os.path.join(fam, "*.json"))):
            if "config" in js:
                continue
            if "ffn" not in fam and ("falcon" in base) != ("falcon" in os.path.basename(js)):
                continue
            hit = next((e for e in json.load(open(js)) if isinstance(e, dict) and e.get("ir_id") == ir_id), None)
            if hit is None:
                continue
            ir = hit["ir_expression"]
            names = set(re.findall(r"\((?:input|output|tensor) ([^()]+)\)", ir))
            names = {n.strip() for grp in names for n in grp.split(",")}
            if not set(tparams) <= names:
                continue
            out.append({"module": os.path.relpath(py, ref), "json": os.path.relpath(js, ref), "ir_id": ir_id,
                        "n_kernels": n_kernels, "tensor_params": tparams, "block_params": bparams, "ir_expression": ir})
            break
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ir_module_params.json")
    json.dump(out, open(dst, "w"), indent=1)
    print("wrote %d pairs to %s" % (len(out), dst))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
