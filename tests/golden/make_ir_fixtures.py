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
    family_sample(ev)


# what each result file's name says its expressions compute (the model fixes the dimensions:
# evaluation/llama_configs.json, falcon_configs.json, ffn/*/tensor_configs.json)
EXPECT = {
    "vanilla": dict(family="attention", variant="vanilla", prenorm=False, qknorm=False),
    "prenorm": dict(family="attention", variant="vanilla", prenorm=True, qknorm=False),
    "qknorm": dict(family="attention", variant="vanilla", prenorm=False, qknorm=True),
    "keyformer": dict(family="attention", variant="keyformer", prenorm=False, qknorm=False),
    "roco": dict(family="attention", variant="roco", prenorm=False, qknorm=False),
    "ffn_llama": dict(family="ffn", falcon_tail=False),
    "ffn_falcon": dict(family="ffn", falcon_tail=True),
}
DIMS = {"llama": {"M": 16, "D": 128, "N": 4096, "P": 1024, "H": 32}, "falcon": {"M": 16, "D": 64, "N": 4544, "P": 1024, "H": 71}}


def family_sample(ev, per_file=6):
    """A spread of the search's expressions per result file (the fastest one, the first whose projection runs
    under its own ploop, and evenly spaced others), each with what the file name says it computes."""
    out = []
    for js in sorted(glob.glob(os.path.join(ev, "*", "*.json")) + glob.glob(os.path.join(ev, "ffn", "*", "*.json"))):
        if "config" in js:
            continue
        data = json.load(open(js))
        rows = [e for e in data if isinstance(e, dict) and e.get("ir_expression")] if isinstance(data, list) else []
        if not rows:
            continue
        fam = os.path.basename(os.path.dirname(js))
        model = "falcon" if "falcon" in js else "llama"
        picks = {0, len(rows) - 1}
        picks.update(range(0, len(rows), max(1, len(rows) // (per_file - 2))))
        timed = [i for i, e in enumerate(rows) if isinstance(e.get("execution_time_ms"), (int, float))]
        if timed:
            picks.add(min(timed, key=lambda i: rows[i]["execution_time_ms"]))
        split = next((i for i, e in enumerate(rows) if e["ir_expression"].count("(ploop ") > 1), None)
        if split is not None:
            picks.add(split)
        for i in sorted(picks)[: per_file + 2]:
            exp = dict(EXPECT[fam])
            if exp["family"] == "attention":
                exp["dims"] = DIMS[model]
            out.append({"json": os.path.relpath(js, os.path.dirname(ev)), "ir_id": rows[i].get("ir_id"), "expect": exp,
                        "ir_expression": rows[i]["ir_expression"]})
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ir_family_sample.json")
    json.dump(out, open(dst, "w"), indent=1)
    print("wrote %d expressions to %s" % (len(out), dst))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
