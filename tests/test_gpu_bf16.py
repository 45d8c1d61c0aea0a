"""GPU parity of the bf16 kernels (the same sources compiled for bf16 elements) against the CPU oracle with
bf16 rounding points.  bf16 is outside the reference (fp16 throughout); tolerances are this build's: 16-bit
outputs rtol = atol = 3e-2 (bf16 carries 8 mantissa bits, three fewer than fp16), fp32 score accumulators 1e-2
relative with the same absolute floor as the fp16 tests."""
import math

import pytest
import torch

import oracle
from trinity_amd import ext
from util import assert_close, attn_inputs, ffn_inputs, gen

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
RTOL = ATOL = 3e-2


def _bf(t):
    return {k: v.float().to(BF) for k, v in t.items()}


def _scores_close(actual, expected, what):
    a, e = actual.double(), expected.double()
    tol = 1e-2 * e.abs() + 1e-3 * e.abs().amax(dim=-1, keepdim=True) + 1e-7
    assert ((a - e).abs() <= tol).all(), what


def test_rmsnorm_bf16(dev):
    g = gen(3)
    x = (torch.randn(300, 4544, generator=g)).to(BF)
    w = (1 + 0.1 * torch.randn(4544, generator=g)).to(BF)
    for rows in (300, 2000):       # block-per-row and wave-per-row kernels
        xx = x[:rows] if rows <= 300 else x.repeat(7, 1)[:rows].contiguous()
        y = torch.zeros(rows, 4544, dtype=BF, device=dev)
        ext.rmsnorm(xx.to(dev), w.to(dev), y, 1e-5)
        torch.cuda.synchronize()
        assert_close(y, oracle.rmsnorm(xx, w, 1e-5, out_dtype=BF), 1e-2, 1e-2, "rmsnorm bf16 %d rows" % rows)


@pytest.mark.parametrize("T,N,F", [(300, 512, 1088), (16, 512, 1088), (2048, 512, 4544)])
def test_ffn_bf16(dev, T, N, F):
    t = _bf(ffn_inputs(T, N, F, w_std=0.05))
    d = {k: v.to(dev) for k, v in t.items()}
    nbytes = ext.ffn_workspace_bytes(T, N, F)
    ws = torch.zeros(max(nbytes, 16), dtype=torch.uint8, device=dev)
    hid = torch.zeros(T, F, dtype=BF, device=dev)
    out = torch.zeros(T, N, dtype=BF, device=dev)
    ext.ffn_swiglu(d["x"], d["w1"], d["w_up"], d["w2"], hid, out, workspace=ws)
    torch.cuda.synchronize()
    want, want_h = oracle.ffn_swiglu(t["x"], t["w1"], t["w_up"], t["w2"], elem=BF)
    assert_close(hid, want_h, RTOL, ATOL, "swiglu hidden bf16")
    assert_close(out, want, RTOL, ATOL, "swiglu out bf16")
    ext.ffn_gelu(d["x"], d["w1"], d["w2"], hid, out, workspace=ws)
    torch.cuda.synchronize()
    want, want_h = oracle.ffn_gelu(t["x"], t["w1"], t["w2"], elem=BF)
    assert_close(hid, want_h, RTOL, ATOL, "gelu hidden bf16")
    assert_close(out, want, RTOL, ATOL, "gelu out bf16")


CASES = [
    # S,  N,   Hq, Hkv, D,  P,  causal
    (192, 256, 4, 2, 128, 0, True),
    (200, 256, 4, 4, 64, 0, True),
    (16, 256, 4, 4, 64, 300, False),     # few-token regime: split-K projection, key-split attention
    (40, 256, 2, 2, 128, 70, True),
    (16, 128, 4, 2, 128, 300, True),     # few tokens, head dimension 128: the projection's own merge kernel
    (16, 128, 4, 2, 128, 4200, True),    # long prefix: the looping key-split kernel, heads stacked
    (20, 128, 6, 1, 64, 2500, False),
]


def _run(t, dev, variant, Hq, Hkv, D, P, scale, causal, **kw):
    S, N = t["x"].shape
    p = ext.attn_params(Hq, Hkv, D, S, kv_prefix=P, scale=scale, causal=causal, rms_eps=1e-5, tau=1.0,
                        noise_seed=kw.get("seed", 0), prenorm=kw.get("prenorm", False), qknorm=kw.get("qknorm", False))
    d = {k: v.to(dev) for k, v in t.items()}
    kc, vc = d.get("k_cache"), d.get("v_cache")
    nw = d["norm_w"] if kw.get("prenorm") else None
    out = torch.zeros(S, Hq * D, dtype=BF, device=dev)
    scratch = torch.empty(ext.qkv_scratch_bytes(p, N), dtype=torch.uint8, device=dev)
    res = {}
    if variant == "vanilla":
        ext.qkv_attention(d["x"], nw, d["wq"], d["wk"], d["wv"], kc, vc, scratch, None, out, p)
    elif variant == "roco":
        s1 = torch.zeros(Hq, P + S, dtype=torch.float32, device=dev)
        s2 = torch.zeros(Hq, P + S, dtype=torch.float32, device=dev)
        ext.roco(d["x"], nw, d["wq"], d["wk"], d["wv"], kc, vc, scratch, out, s1, s2, p)
        res["s1"], res["s2"] = s1.cpu(), s2.cpu()
    else:
        sc = torch.zeros(Hq, P + S, dtype=torch.float32, device=dev)
        ext.keyformer(d["x"], nw, d["wq"], d["wk"], d["wv"], kc, vc, scratch, None, out, sc, p)
        res["score"] = sc.cpu()
    torch.cuda.synchronize()
    res["O2"] = out.cpu()
    if kc is not None:
        res["k_cache"] = kc.cpu()
    return res


@pytest.mark.parametrize("S,N,Hq,Hkv,D,P,causal", CASES)
@pytest.mark.parametrize("variant,prenorm,qknorm", [("vanilla", False, False), ("vanilla", True, False), ("vanilla", False, True),
                                                     ("roco", False, False), ("keyformer", False, False)])
def test_attention_bf16(dev, S, N, Hq, Hkv, D, P, causal, variant, prenorm, qknorm):
    t = _bf(attn_inputs(S, N, Hq, Hkv, D, P=P, w_std=0.06))
    scale = 1.0 / math.sqrt(D)
    want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=scale,
                                causal=causal, kv_prefix=P, k_cache=t.get("k_cache"), v_cache=t.get("v_cache"),
                                prenorm=prenorm, prenorm_weight=t["norm_w"] if prenorm else None, rms_eps=1e-5,
                                qknorm=qknorm, roco=variant == "roco", keyformer=variant == "keyformer", noise_seed=5,
                                tau=1.0, elem=BF)
    got = _run(t, dev, variant, Hq, Hkv, D, P, scale, causal, prenorm=prenorm, qknorm=qknorm, seed=5)
    assert_close(got["O2"], want["O2"], RTOL, ATOL, "O2 bf16")
    if P:
        assert_close(got["k_cache"][:, P:], want["k_new"], RTOL, ATOL, "appended K rows bf16")
    if variant == "roco":
        _scores_close(got["s1"], want["s1"], "s1 bf16")
        _scores_close(got["s2"], want["s2"], "s2 bf16")
    if variant == "keyformer":
        _scores_close(got["score"], want["score"], "score bf16")
