"""GPU: the entry point that allocates nothing (tri_qkv_attention_static, scratch memory in the library's own
per-GPU array) against tri_qkv_attention with caller-provided scratch: same inputs, same outputs, on calls in a
row that share the array - the second with a smaller input, so that it runs over what the first one left."""
import math

import pytest
import torch

from trinity_amd import ext
from util import attn_inputs

pytestmark = pytest.mark.gpu


def _both(dev, S, N, Hq, Hkv, D, P, causal, prenorm=False, qknorm=False, seed=1):
    t = attn_inputs(S, N, Hq, Hkv, D, P=P, seed=seed, w_std=0.05, with_cache=True)
    p = ext.attn_params(Hq, Hkv, D, S, kv_prefix=P, causal=causal, rms_eps=1e-5, prenorm=prenorm, qknorm=qknorm,
                        scale=1.0 / math.sqrt(D))
    d = {k: v.to(dev) for k, v in t.items()}
    nw = d["norm_w"] if prenorm else None
    res = []
    for static in (False, True):
        kc, vc = d["k_cache"].clone(), d["v_cache"].clone()
        out = torch.zeros(S, Hq * D, dtype=torch.float16, device=dev)
        lse = torch.zeros(Hq, S, dtype=torch.float32, device=dev)
        if static:
            ext.qkv_attention_static(d["x"], nw, d["wq"], d["wk"], d["wv"], kc, vc, lse, out, p)
        else:
            scratch = torch.empty(ext.qkv_scratch_bytes(p, N), dtype=torch.uint8, device=dev)
            ext.qkv_attention(d["x"], nw, d["wq"], d["wk"], d["wv"], kc, vc, scratch, lse, out, p)
        torch.cuda.synchronize()
        res.append((out.cpu(), lse.cpu(), kc.cpu(), vc.cpu()))
    return res


# (many tokens: large tiles + prefill attention) then (few tokens: split-K projection + key-split attention), each
# followed by a smaller call of the same kind that reuses the array
CALLS = [
    dict(S=384, N=512, Hq=8, Hkv=2, D=128, P=64, causal=True),
    dict(S=96, N=256, Hq=4, Hkv=4, D=64, P=0, causal=True, prenorm=True),
    dict(S=16, N=512, Hq=8, Hkv=8, D=64, P=600, causal=False, qknorm=True),
    dict(S=5, N=256, Hq=4, Hkv=1, D=128, P=40, causal=True),
]


def test_static_scratch_matches_caller_scratch(dev):
    ext.prepare()
    for i, c in enumerate(CALLS):
        (o_a, l_a, k_a, v_a), (o_b, l_b, k_b, v_b) = _both(dev, seed=10 + i, **c)
        assert torch.isfinite(o_b.float()).all()
        # the same kernels over the same layout at another address: the results are the same bits
        assert torch.equal(o_a, o_b), "O2 differs in call %d" % i
        assert torch.equal(l_a, l_b), "log-sum-exp differs in call %d" % i
        assert torch.equal(k_a, k_b) and torch.equal(v_a, v_b), "appended cache rows differ in call %d" % i


def test_static_scratch_under_graph_capture(dev):
    """What the entry point is for: after tri_prepare, calls of it are captured into a HIP graph on a side stream and
    replayed - the larger call first, then a smaller one that runs over what the first left in the array - and each
    replay equals the eager call with caller-provided scratch; eager calls leave the amount of device memory held
    outside torch's allocator unchanged."""
    ext.prepare()
    cases = []
    for i, c in enumerate((CALLS[0], CALLS[3])):
        S, N, Hq, Hkv, D, P = c["S"], c["N"], c["Hq"], c["Hkv"], c["D"], c["P"]
        t = attn_inputs(S, N, Hq, Hkv, D, P=P, seed=20 + i, w_std=0.05, with_cache=True)
        d = {k: v.to(dev) for k, v in t.items()}
        p = ext.attn_params(Hq, Hkv, D, S, kv_prefix=P, causal=c["causal"], scale=1.0 / math.sqrt(D))
        out = torch.zeros(S, Hq * D, dtype=torch.float16, device=dev)
        lse = torch.zeros(Hq, S, dtype=torch.float32, device=dev)
        kc, vc = d["k_cache"].clone(), d["v_cache"].clone()
        # the eager result with caller-provided scratch
        want_out, want_lse = torch.zeros_like(out), torch.zeros_like(lse)
        kc2, vc2 = d["k_cache"].clone(), d["v_cache"].clone()
        scratch = torch.empty(ext.qkv_scratch_bytes(p, N), dtype=torch.uint8, device=dev)
        ext.qkv_attention(d["x"], None, d["wq"], d["wk"], d["wv"], kc2, vc2, scratch, want_lse, want_out, p)
        cases.append((d, p, out, lse, kc, vc, want_out, want_lse, kc2))
    del scratch
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graphs = []
    for d, p, out, lse, kc, vc, *_ in cases:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            with torch.cuda.graph(g, stream=stream):
                ext.qkv_attention_static(d["x"], None, d["wq"], d["wk"], d["wv"], kc, vc, lse, out, p)
        graphs.append(g)
    stream.synchronize()
    for rep in range(2):
        for (d, p, out, lse, kc, vc, want_out, want_lse, kc2), g in zip(cases, graphs):
            out.fill_(7.0)
            lse.zero_()
            torch.cuda.synchronize()          # eager work and a synchronisation between the replays
            with torch.cuda.stream(stream):
                g.replay()
            stream.synchronize()
            assert torch.equal(out, want_out), "replay %d: O2 differs from the eager call" % rep
            assert torch.equal(lse, want_lse), "replay %d: log-sum-exp differs" % rep
            assert torch.equal(kc, kc2), "replay %d: appended K rows differ" % rep
    # The entry point's host code allocates nothing: over eager calls of it (a replay runs none of the library's
    # host code, and the graph machinery keeps memory of its own) the device memory held outside torch's caching
    # allocator - free + reserved - stays the same.
    outside = lambda: torch.cuda.mem_get_info()[0] + torch.cuda.memory_reserved()
    torch.cuda.synchronize()
    before = outside()
    for d, p, out, lse, kc, vc, *_ in cases + cases:
        ext.qkv_attention_static(d["x"], None, d["wq"], d["wk"], d["wv"], kc, vc, lse, out, p)
    torch.cuda.synchronize()
    assert outside() == before, "device memory outside torch's allocator changed across eager calls"


def test_static_scratch_against_the_oracle(dev):
    import oracle
    from util import assert_close

    c = CALLS[0]
    t = attn_inputs(c["S"], c["N"], c["Hq"], c["Hkv"], c["D"], P=c["P"], seed=3, w_std=0.05, with_cache=True)
    p = ext.attn_params(c["Hq"], c["Hkv"], c["D"], c["S"], kv_prefix=c["P"], causal=True)
    d = {k: v.to(dev) for k, v in t.items()}
    out = torch.zeros(c["S"], c["Hq"] * c["D"], dtype=torch.float16, device=dev)
    ext.qkv_attention_static(d["x"], None, d["wq"], d["wk"], d["wv"], d["k_cache"], d["v_cache"], None, out, p)
    torch.cuda.synchronize()
    want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], n_q_heads=c["Hq"], n_kv_heads=c["Hkv"],
                                head_dim=c["D"], scale=1 / math.sqrt(c["D"]), causal=True, kv_prefix=c["P"],
                                k_cache=t["k_cache"], v_cache=t["v_cache"])
    assert_close(out, want["O2"], 1e-2, 1e-2, "O2 through the static scratch array")   # fp16 outputs: rtol = atol = 1e-2


def test_static_scratch_refuses_what_does_not_fit(dev):
    # Llama-3-8B heads, 8192 new tokens: the scratch layout needs more than the array holds -> refused, nothing runs
    S, N, Hq, Hkv, D = 8192, 4096, 32, 8, 128
    p = ext.attn_params(Hq, Hkv, D, S, causal=True)
    assert ext.qkv_scratch_bytes(p, N) > ext.STATIC_SCRATCH_BYTES
    x = torch.zeros(S, N, dtype=torch.float16, device=dev)
    w = torch.zeros(N, Hq * D, dtype=torch.float16, device=dev)
    wkv = torch.zeros(N, Hkv * D, dtype=torch.float16, device=dev)
    out = torch.full((S, Hq * D), 7.0, dtype=torch.float16, device=dev)
    assert ext.qkv_attention_static(x, None, w, wkv, wkv, None, None, None, out, p, status_only=True) == -7
    torch.cuda.synchronize()
    assert (out == 7).all()
