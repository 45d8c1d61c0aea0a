"""GPU parity with KV caches held as fp8 (OCP e4m3, one fp32 scale per tensor), through the C ABI against the
CPU oracle: the appended rows are fp8(k / k_scale), fp8(v / v_scale) and attention sees scale * fp8 for every
key.  The reference has no fp8 cache; the oracle's definition (torch.float8_e4m3fn casts) is the bar.

Tolerances: fp16 outputs rtol = atol = 1e-2, fp32 scores 1e-3.  The appended fp8 codes are compared exactly; a
code may differ by one step where the projection's fp16 rounding (kernel: fp32 accumulation in a different
order) lands on the other side of an fp8 rounding boundary - at most 1 % of the entries."""
import math

import pytest
import torch

import oracle
from gpu_util import scratch_for
from test_gpu_attention import assert_scores
from trinity_amd import ext
from util import assert_close, attn_inputs, gen

pytestmark = pytest.mark.gpu
F8 = torch.float8_e4m3fn
K_SCALE, V_SCALE = 0.04, 0.015


def _fp8_inputs(S, N, Hq, Hkv, D, P, dtype=torch.float16):
    t = attn_inputs(S, N, Hq, Hkv, D, P=P, w_std=0.06, with_cache=True)
    t = {k: (v.to(dtype) if v.dtype == torch.float16 else v) for k, v in t.items()}
    kc = (t["k_cache"].float() / K_SCALE).clamp(-448, 448).to(F8)
    vc = (t["v_cache"].float() / V_SCALE).clamp(-448, 448).to(F8)
    kc[:, P:] = torch.zeros_like(kc[:, P:])
    vc[:, P:] = torch.zeros_like(vc[:, P:])
    t["k_cache"], t["v_cache"] = kc, vc
    return t


def _codes_match(got, want, what):
    g, w = got.view(torch.uint8).int(), want.view(torch.uint8).int()
    diff = (g - w).abs()
    frac = (diff != 0).float().mean().item()
    assert frac <= 0.01, "%s: %.3f %% of the fp8 codes differ" % (what, 100 * frac)
    one_step = (diff <= 1) | (((g & 0x7F) + (w & 0x7F)) <= 1)  # neighbours, or +-0 against the smallest value
    assert bool(one_step.all()), what + ": a code differs by more than one step"


def _run(t, dev, variant, *, Hq, Hkv, D, P, causal, qknorm=False, seed=0, tau=1.0, dtype=torch.float16):
    S, N = t["x"].shape
    p = ext.attn_params(Hq, Hkv, D, S, kv_prefix=P, causal=causal, qknorm=qknorm, rms_eps=1e-5, tau=tau,
                        noise_seed=seed, kv_fp8=True, k_scale=K_SCALE, v_scale=V_SCALE)
    d = {k: v.to(dev) for k, v in t.items()}
    out = torch.zeros(S, Hq * D, dtype=dtype, device=dev)
    scratch = scratch_for(p, N, dev)
    res = {}
    if variant == "vanilla":
        ext.qkv_attention(d["x"], None, d["wq"], d["wk"], d["wv"], d["k_cache"], d["v_cache"], scratch, None, out, p)
    elif variant == "roco":
        s1 = torch.zeros(Hq, P + S, dtype=torch.float32, device=dev)
        s2 = torch.zeros(Hq, P + S, dtype=torch.float32, device=dev)
        ext.roco(d["x"], None, d["wq"], d["wk"], d["wv"], d["k_cache"], d["v_cache"], scratch, out, s1, s2, p)
        res["s1"], res["s2"] = s1.cpu(), s2.cpu()
    else:
        score = torch.zeros(Hq, P + S, dtype=torch.float32, device=dev)
        ext.keyformer(d["x"], None, d["wq"], d["wk"], d["wv"], d["k_cache"], d["v_cache"], scratch, None, out, score, p)
        res["score"] = score.cpu()
    torch.cuda.synchronize()
    res["O2"] = out.cpu()
    res["k_cache"], res["v_cache"] = d["k_cache"].cpu(), d["v_cache"].cpu()
    return res


CASES = [
    # S,  N,   Hq, Hkv, D,  P,   causal
    (16, 256, 4, 2, 128, 1024, False),   # the reference's regime: the kernel reads the fp8 rows itself
    (32, 256, 2, 2, 64, 500, True),
    (5, 128, 2, 1, 64, 253, True),       # ragged
    (1, 128, 4, 4, 128, 0, True),        # nothing cached yet
    (100, 256, 4, 2, 128, 60, True),     # more tokens: through the 16-bit copy
    (200, 320, 5, 1, 64, 0, True),
    (16, 128, 4, 2, 128, 4200, True),    # long prefix: the looping key-split kernel converts the fp8 tiles itself
    (20, 128, 6, 1, 64, 3001, False),    # ... 120 stacked rows, ragged last tile
]


@pytest.mark.parametrize("S,N,Hq,Hkv,D,P,causal", CASES)
@pytest.mark.parametrize("qknorm", [False, True])
def test_fp8_cache_vanilla(dev, S, N, Hq, Hkv, D, P, causal, qknorm):
    t = _fp8_inputs(S, N, Hq, Hkv, D, P)
    kw = dict(n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=1 / math.sqrt(D), causal=causal, kv_prefix=P,
              k_cache=t["k_cache"], v_cache=t["v_cache"], kv_fp8=True, k_scale=K_SCALE, v_scale=V_SCALE)
    want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], qknorm=qknorm, rms_eps=1e-5, **kw)
    got = _run(t, dev, "vanilla", Hq=Hq, Hkv=Hkv, D=D, P=P, causal=causal, qknorm=qknorm)
    _codes_match(got["k_cache"][:, P:P + S], want["k_new"], "appended k")
    _codes_match(got["v_cache"][:, P:P + S], want["v_new"], "appended v")
    assert torch.equal(got["k_cache"][:, :P].view(torch.uint8), t["k_cache"][:, :P].view(torch.uint8))
    assert torch.equal(got["v_cache"][:, :P].view(torch.uint8), t["v_cache"][:, :P].view(torch.uint8))
    assert_close(got["O2"], want["O2"], 1e-2, 1e-2, "O2")


@pytest.mark.parametrize("S,N,Hq,Hkv,D,P,causal", [CASES[0], CASES[2], CASES[4], CASES[6]])
def test_fp8_cache_scores(dev, S, N, Hq, Hkv, D, P, causal):
    t = _fp8_inputs(S, N, Hq, Hkv, D, P)
    kw = dict(n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=1 / math.sqrt(D), causal=causal, kv_prefix=P,
              k_cache=t["k_cache"], v_cache=t["v_cache"], kv_fp8=True, k_scale=K_SCALE, v_scale=V_SCALE)
    # the fp32 score accumulators are held to 1e-3, finer than one flipped fp8 code allows: the appended rows are
    # checked on their own and the attention part against the cache contents the library produced
    got = _run(t, dev, "roco", Hq=Hq, Hkv=Hkv, D=D, P=P, causal=causal)
    rows = (got["k_cache"][:, P:P + S], got["v_cache"][:, P:P + S])
    want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], roco=True, appended_fp8=rows, **kw)
    _codes_match(rows[0], want["k_new"], "appended k")
    _codes_match(rows[1], want["v_new"], "appended v")
    assert_close(got["O2"], want["O2"], 1e-2, 1e-2, "roco O2")
    assert_scores(got["s1"], want["s1"], "s1")
    assert_scores(got["s2"], want["s2"], "s2")
    got = _run(t, dev, "keyformer", Hq=Hq, Hkv=Hkv, D=D, P=P, causal=causal, seed=9)
    rows = (got["k_cache"][:, P:P + S], got["v_cache"][:, P:P + S])
    want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], keyformer=True, noise_seed=9, tau=1.0,
                                appended_fp8=rows, **kw)
    assert_close(got["O2"], want["O2"], 1e-2, 1e-2, "keyformer O2")
    assert_scores(got["score"], want["score"], "score")


def test_fp8_cache_bf16_elements(dev):
    S, N, Hq, Hkv, D, P = 16, 256, 4, 2, 128, 300
    t = _fp8_inputs(S, N, Hq, Hkv, D, P, dtype=torch.bfloat16)
    want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D,
                                scale=1 / math.sqrt(D), causal=False, kv_prefix=P, k_cache=t["k_cache"],
                                v_cache=t["v_cache"], kv_fp8=True, k_scale=K_SCALE, v_scale=V_SCALE,
                                elem=torch.bfloat16)
    got = _run(t, dev, "vanilla", Hq=Hq, Hkv=Hkv, D=D, P=P, causal=False, dtype=torch.bfloat16)
    assert_close(got["O2"], want["O2"], 3e-2, 3e-2, "O2 (bf16 elements)")
    _codes_match(got["k_cache"][:, P:P + S], want["k_new"], "appended k")
