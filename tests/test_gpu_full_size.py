"""GPU parity at the benchmark configurations' full sizes.

The device runs the whole problem; the CPU oracle checks a sample of query
heads (heads are independent given X and the weights), and size-independent
properties cover everything: the first causal query attends to key 0 only, the
per-key probability masses sum to S per head, mean/variance relate to the raw
sums, outputs are finite."""
import math

import pytest
import torch

import oracle
from gpu_util import run_qkv
from util import assert_close, attn_inputs

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def _subset(t, heads, Hq, Hkv, D):
    """Reduced problem holding only `heads`: each selected query head gets its own copy of its KV head."""
    grp = Hq // Hkv
    qcols = torch.cat([torch.arange(h * D, (h + 1) * D) for h in heads])
    kcols = torch.cat([torch.arange((h // grp) * D, (h // grp + 1) * D) for h in heads])
    r = {"x": t["x"], "wq": t["wq"][:, qcols].contiguous(), "wk": t["wk"][:, kcols].contiguous(),
         "wv": t["wv"][:, kcols].contiguous(), "norm_w": t["norm_w"]}
    return r, qcols


def _check_projection(got, t, Hq, Hkv, D, prenorm=False, qknorm=False, eps=0.0):
    """Every column of the Q / K / V projection (so every tile of whatever tile plan the launch took, including
    the narrower tiles of a plan's last columns) against an fp32 product on the CPU; the normalisations are the
    oracle's rmsnorm.  `got` comes from a call with caches (K / V rows land in them) and keep_scratch (the scratch
    buffer starts with the q rows [S, Hq * D])."""
    S = t["x"].shape[0]
    x = oracle.rmsnorm(t["x"], t["norm_w"], eps) if prenorm else t["x"]
    xf = x.float()
    q = (xf @ t["wq"].float()).half()
    k = (xf @ t["wk"].float()).half()
    v = (xf @ t["wv"].float()).half()
    if qknorm:
        q = oracle.rmsnorm(q.view(S * Hq, D), None, eps).view(S, Hq * D)
        k = oracle.rmsnorm(k.view(S * Hkv, D), None, eps).view(S, Hkv * D)
    q_dev = got["scratch"][: S * Hq * D * 2].view(torch.float16).view(S, Hq * D)
    assert_close(q_dev, q, RTOL, ATOL, "q, all heads")
    assert_close(got["k_cache"].transpose(0, 1).reshape(S, Hkv * D), k, RTOL, ATOL, "k, all heads")
    assert_close(got["v_cache"].transpose(0, 1).reshape(S, Hkv * D), v, RTOL, ATOL, "v, all heads")


def _check_scores(got, want, what):
    a, e = got.double(), want.double()
    tol = 1e-3 * e.abs() + 1e-4 * e.abs().amax(dim=-1, keepdim=True) + 1e-7
    bad = (a - e).abs() > tol
    assert not bad.any(), "%s: %d entries beyond 1e-3 relative" % (what, int(bad.sum()))


@pytest.mark.parametrize("S", [1024, 4096])
def test_vanilla_llama(dev, S):
    N, Hq, Hkv, D = 4096, 32, 8, 128
    t = attn_inputs(S, N, Hq, Hkv, D, with_cache=True)
    scale = 1.0 / math.sqrt(D)
    got = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, scale=scale, causal=True, want_lse=True, keep_scratch=True)
    assert torch.isfinite(got["O2"]).all()
    _check_projection(got, t, Hq, Hkv, D)
    heads = [0, 13, 31] if S > 1024 else list(range(0, 32, 5))
    sub, qcols = _subset(t, heads, Hq, Hkv, D)
    want = oracle.qkv_attention(sub["x"], sub["wq"], sub["wk"], sub["wv"], n_q_heads=len(heads), n_kv_heads=len(heads),
                                head_dim=D, scale=scale, causal=True, want_lse=True, head_chunk=1)
    assert_close(got["O2"][:, qcols], want["O2"], RTOL, ATOL, "O2 heads %s" % heads)
    assert_close(got["lse"][heads], want["lse"], 1e-3, 2e-3, "lse")
    # query 0 sees key 0 only: its output row is v[0] of its KV head, exactly
    v0 = (t["x"][:1].float() @ t["wv"].float()).half().view(Hkv, D)
    o0 = got["O2"][0].view(Hq, D)
    assert_close(o0, v0.repeat_interleave(Hq // Hkv, dim=0), 2e-3, 2e-3, "first causal row")


@pytest.mark.parametrize("S", [1024, 4096])
@pytest.mark.parametrize("prenorm,qknorm", [(True, False), (False, True)])
def test_prenorm_qknorm_falcon(dev, S, prenorm, qknorm):
    N, Hq, Hkv, D = 4544, 71, 1, 64
    t = attn_inputs(S, N, Hq, Hkv, D, with_cache=True)
    scale = 1.0 / math.sqrt(D)
    got = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, scale=scale, causal=True, prenorm=prenorm, qknorm=qknorm, eps=1e-5,
                  keep_scratch=True)
    assert torch.isfinite(got["O2"]).all()
    _check_projection(got, t, Hq, Hkv, D, prenorm=prenorm, qknorm=qknorm, eps=1e-5)
    heads = [0, 35, 70]
    sub, qcols = _subset(t, heads, Hq, Hkv, D)
    want = oracle.qkv_attention(sub["x"], sub["wq"], sub["wk"], sub["wv"], n_q_heads=3, n_kv_heads=3, head_dim=D,
                                scale=scale, causal=True, prenorm=prenorm, prenorm_weight=t["norm_w"], rms_eps=1e-5,
                                qknorm=qknorm, head_chunk=1)
    assert_close(got["O2"][:, qcols], want["O2"], RTOL, ATOL, "O2")


@pytest.mark.parametrize("S", [2048, 4096])
def test_roco_llama(dev, S):
    N, Hq, Hkv, D = 4096, 32, 8, 128
    t = attn_inputs(S, N, Hq, Hkv, D)
    scale = 1.0 / math.sqrt(D)
    got = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, scale=scale, causal=True, variant="roco")
    mv = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, scale=scale, causal=True, variant="roco", mean_var=True)
    heads = [3, 20]
    sub, qcols = _subset(t, heads, Hq, Hkv, D)
    want = oracle.qkv_attention(sub["x"], sub["wq"], sub["wk"], sub["wv"], n_q_heads=2, n_kv_heads=2, head_dim=D,
                                scale=scale, causal=True, roco=True, head_chunk=1)
    assert_close(got["O2"][:, qcols], want["O2"], RTOL, ATOL, "O2")
    _check_scores(got["s1"][heads], want["s1"], "s1")
    _check_scores(got["s2"][heads], want["s2"], "s2")
    # all heads: every query row sums to one, so the per-key masses sum to S; the last key is seen by one query only
    assert torch.allclose(got["s1"].sum(-1), torch.full((Hq,), float(S)), rtol=2e-4)
    assert (got["s2"] <= got["s1"] * (1 + 1e-5) + 1e-7).all()
    assert torch.allclose(got["s2"][:, -1], got["s1"][:, -1] ** 2, rtol=1e-4)
    mean = got["s1"] / S
    assert torch.allclose(mv["s1"], mean, rtol=1e-5, atol=1e-9)
    assert torch.allclose(mv["s2"], got["s2"] / S - mean ** 2, rtol=1e-3, atol=1e-7)


@pytest.mark.parametrize("S", [2048, 4096])
def test_keyformer_llama(dev, S):
    N, Hq, Hkv, D = 4096, 32, 8, 128
    t = attn_inputs(S, N, Hq, Hkv, D)
    scale = 1.0 / math.sqrt(D)
    got = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, scale=scale, causal=True, variant="keyformer", seed=42, tau=1.0)
    heads = [7, 18] if S > 2048 else [7, 30]     # two KV groups either way
    sub, qcols = _subset(t, heads, Hq, Hkv, D)
    want = oracle.qkv_attention(sub["x"], sub["wq"], sub["wk"], sub["wv"], n_q_heads=len(heads), n_kv_heads=len(heads),
                                head_dim=D, scale=scale, causal=True, keyformer=True, noise_seed=42, tau=1.0,
                                noise_head_ids=heads, head_chunk=1)
    assert_close(got["O2"][:, qcols], want["O2"], RTOL, ATOL, "O2")
    _check_scores(got["score"][heads], want["score"], "score")
    assert torch.allclose(got["score"].sum(-1), torch.full((Hq,), float(S)), rtol=2e-4)
    # a different seed changes the scores but not the attention output
    other = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, scale=scale, causal=True, variant="keyformer", seed=43, tau=1.0)
    assert torch.equal(other["O2"], got["O2"])
    assert not torch.allclose(other["score"], got["score"], rtol=1e-2)


@pytest.mark.parametrize("variant", ["vanilla", "roco", "keyformer"])
def test_few_tokens_long_prefix_llama(dev, variant):
    """16 new tokens against 32768 cached keys with Llama-3-8B's heads (32 over 8 KV heads): the looping key-split
    kernel at its real shape, every output checked against the oracle (16 queries make that cheap)."""
    S, N, Hq, Hkv, D, P = 16, 4096, 32, 8, 128, 32768
    t = attn_inputs(S, N, Hq, Hkv, D, P=P, w_std=0.02)
    scale = 1.0 / math.sqrt(D)
    kw = dict(n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=scale, causal=True, kv_prefix=P,
              k_cache=t["k_cache"], v_cache=t["v_cache"])
    if variant == "vanilla":
        want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], want_lse=True, **kw)
        got = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, P=P, scale=scale, causal=True, want_lse=True)
        assert_close(got["lse"], want["lse"], 1e-3, 2e-3, "lse")
        assert_close(got["k_cache"][:, P:], want["k_new"], RTOL, ATOL, "k rows")
        assert torch.equal(got["k_cache"][:, :P], t["k_cache"][:, :P])
    elif variant == "roco":
        want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], roco=True, **kw)
        got = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, P=P, scale=scale, causal=True, variant="roco")
        _check_scores(got["s1"], want["s1"], "sum p")
        _check_scores(got["s2"], want["s2"], "sum p^2")
        # every query's probabilities sum to one: the per-key masses of a head add up to the number of queries
        assert torch.allclose(got["s1"].double().sum(-1), torch.full((Hq,), float(S), dtype=torch.float64), rtol=1e-4)
    else:
        want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], keyformer=True, noise_seed=9, tau=1.0, **kw)
        got = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, P=P, scale=scale, causal=True, variant="keyformer", seed=9, tau=1.0)
        _check_scores(got["score"], want["score"], "score")
    assert_close(got["O2"], want["O2"], RTOL, ATOL, "O2")
