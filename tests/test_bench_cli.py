"""bench.py's command line where no GPU is needed: more than one GPU is refused with a message, and without a GPU
the script fails instead of printing a number."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300, cwd=ROOT)


def test_more_than_one_gpu_is_refused():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "--gpus 1" in (r.stdout + r.stderr)
    assert "{" not in r.stdout                      # no result line


def test_no_gpu_no_number():
    import torch
    if torch.cuda.is_available():
        return                                      # (covered by the GPU run of bench.py itself)
    r = _run("--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "{" not in r.stdout


def test_bounds_from_committed_counters():
    """The issue-bound and power-bound estimates are host arithmetic over the instruction counts in the committed
    counter summary: every softmax block of the table gets both, from a model with round numbers, and the bounds
    are what the formulas in the models' notes say."""
    sys.path.insert(0, ROOT)
    import bench

    inputs = bench._issue_inputs()
    names = ["vanilla_llama3_8b_S1024", "vanilla_llama3_8b_S4096", "prenorm_falcon7b_S1024", "prenorm_falcon7b_S4096",
             "qknorm_falcon7b_S1024", "qknorm_falcon7b_S4096", "keyformer_llama3_8b_S2048", "keyformer_llama3_8b_S4096",
             "roco_llama3_8b_S2048", "roco_llama3_8b_S4096"]
    for n in names:
        kinds = [k["kind"] for k in inputs[n]]
        assert kinds[:2] == ["proj", "attn"] and (("score" in kinds) == n.startswith(("keyformer", "roco")))
        assert all(k["insts_lds"] > 0 and k["insts_mfma"] > 0 and k["us"] > 0 for k in inputs[n])
    blocks = [{"block": n, "us": 1000.0} for n in names] + [{"block": "rmsnorm_4096x4096", "us": 10.0}]
    issue = {"mfma": 32.0, "valu": 3.0, "free": 4.0, "trans": 8.0}
    power = {"mfma_ns": 20.0, "lds_read_ns": 2.0, "valu_ns": 0.5, "trans_ns": 1.5, "dma_load_ns": 10.0}
    bench.add_issue_bounds(blocks, issue)
    bench.add_power_bounds(blocks, power)
    assert "issue_bound_us" not in blocks[-1] and "power_bound_us" not in blocks[-1]
    for b in blocks[:-1]:
        assert 0.0 < b["issue_bound_us"] <= b["kernels_us_under_counters"] * 1.5
        assert abs(sum(b["power_bound_parts_us"].values()) - b["power_bound_us"]) < 0.2
        assert abs(b["frac_of_power_bound"] - b["power_bound_us"] / 1000.0) < 1e-12
    # one kernel by hand: the RoCo score pass at S = 4096
    k = [k for k in inputs["roco_llama3_8b_S4096"] if k["kind"] == "score"][0]
    m, t, l = k["insts_mfma"], k["insts_trans"], k["insts_lds"]
    v = k["insts_valu"] - m - t
    want = (20.0 * m + 2.0 * l + 0.5 * v + 1.5 * t + 10.0 * m / 4) / 1024.0 * 1e-3
    got = [b for b in blocks if b["block"] == "roco_llama3_8b_S4096"][0]["power_bound_parts_us"]["score"]
    assert abs(got - want) < 0.06
