"""Front end (no GPU): IR parser, structural analysis, family recognition and
the generated-module protocol."""
import inspect
import json
import os

import pytest

from trinity_amd.codegen import IRParser, NodeType, convert_ir_to_triton
from trinity_amd.codegen.analysis import analyse, flatten_seq
from trinity_amd.codegen.recognise import UnsupportedIR, recognise
from trinity_amd.evaluation import cases

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ir_module_params.json")


def test_tokenizer_and_atoms():
    p = IRParser()
    assert p.tokenize("(load (input X) ; comment\n (index fulltile (tile k)))") == [
        "(", "load", "(", "input", "X", ")", "(", "index", "fulltile", "(", "tile", "k", ")", ")", ")"]
    n = p.parse("(x (load (tensor A,B,C) (index (elem n) fulltile)) 1.5)")
    assert n.node_type == NodeType.MUL
    load, lit = n.children
    assert [c.value for c in load.children[0].children] == ["A", "B", "C"]
    assert load.children[1].children[1].node_type == NodeType.FULLTILE
    assert lit.node_type == NodeType.VAR and lit.value == "1.5"          # non-integer literals stay symbolic
    assert p.parse("(ploop 0 4096 128 n dummy)").children[4].node_type == NodeType.DUMMY
    assert p.parse("-3").value == -3


@pytest.mark.parametrize("bad", ["", "(frobnicate 1 2)", "(seq (load (input X) (index fulltile))", "(seq a b) c", ")"])
def test_parser_rejects(bad):
    with pytest.raises(ValueError):
        IRParser().parse(bad)


def test_flatten_seq_drops_dummy_only_entries():
    root = IRParser().parse("(seq (ploop 0 8 4 n (sloop 0 8 tile_p p dummy)) (seq dummy (store (output A) (load (input B) (index fulltile)) (index fulltile))))")
    ks = flatten_seq(root)
    assert len(ks) == 1 and ks[0].node_type == NodeType.STORE


def test_metadata_matches_reference_generated_modules():
    """TENSOR_PARAMS / BLOCK_PARAMS for the reference's own IRs equal the lists its
    generator wrote into the checked-in modules (fixture built by golden/make_ir_fixtures.py)."""
    pairs = json.load(open(GOLDEN))
    assert len(pairs) >= 20
    # ir_ids are reused across sweeps of the Falcon FFN, so a few fixtures pair a module with the IR of
    # another sweep; those are recognisable by a kernel-count mismatch and are skipped
    checked = mismatched = 0
    wrong = []
    for e in pairs:
        info = analyse(IRParser().parse(e["ir_expression"]))
        if len(info.kernels) != e["n_kernels"]:
            continue
        checked += 1
        if info.tensor_params != e["tensor_params"] or info.block_params != e["block_params"]:
            mismatched += 1
            wrong.append(e["module"])
    assert checked >= 20
    # every attention family and the Llama FFN must match exactly
    assert not [w for w in wrong if "ffn_falcon" not in w], wrong
    assert mismatched <= 4, wrong


@pytest.mark.parametrize("variant,pre,qk", [("vanilla", False, False), ("vanilla", True, False), ("vanilla", False, True),
                                              ("vanilla", True, True), ("keyformer", False, False), ("keyformer", True, False),
                                              ("roco", False, False), ("roco", True, False)])
def test_recognise_attention_families(variant, pre, qk):
    for (M, N, D, P, H) in [(16, 4096, 128, 1024, 32), (16, 4544, 64, 1024, 71)]:
        info = analyse(IRParser().parse(cases.attention_ir(variant, M, N, D, P, pre, qk)))
        c = recognise(info)
        assert (c.family, c.variant, c.prenorm, c.qknorm) == ("attention", variant, pre, qk)
        assert c.dims == {"M": M, "N": N, "D": D, "P": P, "H": H}
        assert c.tau == 1.5 if variant == "keyformer" else True
        assert info.block_params == ["block_k", "block_p"]


def test_recognise_reference_irs_from_fixture():
    fam = {"vanilla": ("vanilla", False, False), "prenorm": ("vanilla", True, False), "qknorm": ("vanilla", False, True),
           "keyformer": ("keyformer", False, False), "roco": ("roco", False, False)}
    seen = set()
    for e in json.load(open(GOLDEN)):
        info = analyse(IRParser().parse(e["ir_expression"]))
        c = recognise(info)
        top = e["module"].split("/")[1]
        if top in fam:
            assert (c.variant, c.prenorm, c.qknorm) == fam[top], e["module"]
            assert c.dims["D"] == 64 and c.dims["H"] == 71 and c.dims["P"] == 1024 and c.dims["M"] == 16
            seen.add(top)
        else:
            assert c.family == "ffn"
            assert c.falcon_tail == ("ffn_falcon" in e["module"])
    assert {"prenorm", "qknorm", "keyformer", "roco"} <= seen


def test_unsupported_ir_is_refused():
    ir = "(ploop 0 64 tile_n n (store (output B) (exp (load (input A) (index fulltile (tile n)))) (index fulltile (tile n))))"
    with pytest.raises(UnsupportedIR):
        convert_ir_to_triton(ir)


def _load(src):
    ns = {}
    exec(compile(src, "<generated>", "exec"), ns)
    return ns


def test_generated_module_protocol():
    consts = {"M": 16, "D": 128, "N": 4096, "P": 1024, "H": 32}
    ns = _load(convert_ir_to_triton(cases.attention_ir("keyformer", 16, 4096, 128, 1024), None, consts))
    assert ns["TENSOR_PARAMS"] == sorted(ns["TENSOR_PARAMS"])
    assert ns["TENSOR_PARAMS"] == ["C_exp_perturb", "C_out", "K_cache", "O2", "V_cache", "WK", "WQ", "WV", "X", "noise"]
    assert ns["BLOCK_PARAMS"] == ["block_k", "block_p"]
    sig = inspect.signature(ns["forward"])
    assert list(sig.parameters) == ns["TENSOR_PARAMS"] + ns["BLOCK_PARAMS"]
    assert all(sig.parameters[b].default == 16 for b in ns["BLOCK_PARAMS"])
    plan = ns["_PLAN"]
    assert (plan.variant, plan.M, plan.N, plan.D, plan.H, plan.P, plan.tau) == ("keyformer", 16, 4096, 128, 32, 1024, 1.5)
    assert (plan.scale, plan.causal) == (1.0, False)      # the reference's semantics are the default
    ns = _load(convert_ir_to_triton(cases.ffn_ir(4096, 14336)))
    assert ns["TENSOR_PARAMS"] == ["FF1", "FF2", "O2", "WFF1a", "WFF1b", "WFF2", "WO", "X", "attn_O2"]
    assert ns["BLOCK_PARAMS"] == ["block_k", "block_n", "block_p"]
    ns = _load(convert_ir_to_triton(cases.rmsnorm_ir(4544)))
    assert ns["TENSOR_PARAMS"] == ["O_FF", "O_FF1", "O_FF_norm"]


def test_constants_override_ir_dims():
    ns = _load(convert_ir_to_triton(cases.attention_ir("vanilla", 16, 4096, 128, 1024), None, {"M": 16, "P": 1024, "H": 32}))
    assert ns["_PLAN"].H == 32


def test_configs_keep_reference_keys():
    from trinity_amd.evaluation import harness
    for name in ("llama_configs.json", "falcon_configs.json", "ffn_llama_tensor_configs.json", "ffn_falcon_tensor_configs.json"):
        cfg = harness.load_config(name)
        assert isinstance(cfg, list) and set(cfg[0]) == {"M", "D", "N", "P", "H"}
    assert harness.load_config("llama_configs.json")[0] == {"M": 16, "D": 128, "N": 4096, "P": 1024, "H": 32}
    assert harness.load_config("falcon_configs.json")[0] == {"M": 16, "D": 64, "N": 4544, "P": 1024, "H": 71}
    b = harness.load_config("baseline_configs.json")
    assert b["attention_llama"]["HKV"] == 8 and b["attention_falcon"]["HKV"] == 1


FAMILY_SAMPLE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ir_family_sample.json")


def test_search_expressions_are_recognised_as_what_their_result_file_says():
    """A spread of the expressions the reference's search recorded (evaluation/**/*.json `ir_expression`,
    14,535 in all; tests/golden/make_ir_fixtures.py picks ~6 per file, among them the fastest one and one whose
    projection runs under its own ploop): each must be recognised as the computation its result file is named
    after, with the model's dimensions, and must convert to a module."""
    rows = json.load(open(FAMILY_SAMPLE))
    assert len(rows) > 80
    seen = set()
    for row in rows:
        info = analyse(IRParser().parse(row["ir_expression"]))
        comp = recognise(info, None)
        exp = row["expect"]
        where = "%s ir_id %s" % (row["json"], row["ir_id"])
        assert comp.family == exp["family"], where
        if comp.family == "attention":
            assert (comp.variant, comp.prenorm, comp.qknorm) == (exp["variant"], exp["prenorm"], exp["qknorm"]), where
            assert {k: comp.dims[k] for k in ("M", "N", "D", "P", "H")} == exp["dims"], where
        else:
            assert comp.falcon_tail == exp["falcon_tail"], where
        src = convert_ir_to_triton(row["ir_expression"], None, None)
        assert "def forward(" in src and "TENSOR_PARAMS" in src, where
        seen.add((comp.family, comp.variant, comp.prenorm, comp.qknorm, comp.falcon_tail))
    assert len(seen) == 7


def test_sweep_driver_converts_an_ir_list(tmp_path):
    """The sweep driver reads the reference's `<id>: <expression>` list format, honours --start / --num and
    writes one record per expression with the reference's result fields (no GPU: --convert-only)."""
    from trinity_amd.evaluation import sweep

    rows = [r for r in json.load(open(FAMILY_SAMPLE)) if r["json"].startswith("evaluation/roco/roco_llama")][:4]
    lst = tmp_path / "cases.txt"
    lst.write_text("".join("%d: %s\n" % (100 + i, r["ir_expression"]) for i, r in enumerate(rows)) + "999: dummydata\nnoise line\n")
    assert [i for i, _ in sweep.parse_ir_file(str(lst))] == [100, 101, 102, 103]
    out = tmp_path / "res.json"
    assert sweep.main(["--ir", str(lst), "--m", "llama", "--output", str(out), "--start", "101", "--num", "2", "--convert-only"]) == 0
    res = json.load(open(out))
    assert [r["ir_id"] for r in res] == [101, 102]
    assert set(res[0]) == {"ir_id", "ir_expression", "execution_time_ms", "tensor_config", "error"}
    assert res[0]["tensor_config"] == {"M": 16, "D": 128, "N": 4096, "P": 1024, "H": 32}
    # a result JSON is accepted as an IR list too
    assert [i for i, _ in sweep.parse_ir_file(str(out))] == [101, 102]


def test_run_baseline_refuses_third_party_stacks():
    from trinity_amd.evaluation import run_baseline

    for b in ("trt", "flashinfer", "inductor", "nonsense"):
        with pytest.raises(SystemExit):
            run_baseline.main(["--b", b])
