"""Row strides: every 2-D tensor of a call may be a column slice of a wider buffer (row stride > columns, a
multiple of 8 elements), caches may have padded rows and heads.  Same results as with contiguous tensors, and
nothing outside the slices is written."""
import math

import pytest
import torch

import oracle
from gpu_util import scratch_for
from trinity_amd import ext
from util import assert_close, attn_inputs, ffn_inputs

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2
CANARY = 7.0


def _wide(t, dev, pad=24, fill=CANARY):
    """t placed in the middle columns of a wider buffer: returns (view, buffer)."""
    rows, cols = t.shape
    buf = torch.full((rows, cols + 2 * pad), fill, dtype=t.dtype, device=dev)
    view = buf[:, pad:pad + cols]
    view.copy_(t.to(dev))
    return view, buf


def _untouched(buf, cols, pad=24):
    left, right = buf[:, :pad], buf[:, pad + cols:]
    return bool((left == CANARY).all()) and bool((right == CANARY).all())


@pytest.mark.parametrize("T,N,F,with_ws", [(300, 256, 544, False), (16, 256, 512, True), (40, 320, 256, True)])
def test_ffn_strided(dev, T, N, F, with_ws):
    t = ffn_inputs(T, N, F, w_std=0.05)
    x, xb = _wide(t["x"], dev)
    wg, _ = _wide(t["w1"], dev)
    wu, _ = _wide(t["w_up"], dev)
    wd, _ = _wide(t["w2"], dev)
    hid, hb = _wide(torch.zeros(T, F, dtype=torch.float16), dev)
    out, ob = _wide(torch.zeros(T, N, dtype=torch.float16), dev)
    nbytes = ext.ffn_workspace_bytes(T, N, F) if with_ws else 0
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev) if nbytes else None
    ext.ffn_swiglu(x, wg, wu, wd, hid, out, workspace=ws)
    torch.cuda.synchronize()
    want, want_h = oracle.ffn_swiglu(t["x"], t["w1"], t["w_up"], t["w2"])
    assert_close(hid, want_h, RTOL, ATOL, "hidden")
    assert_close(out, want, RTOL, ATOL, "out")
    assert _untouched(hb, F) and _untouched(ob, N) and _untouched(xb, N)
    hid.zero_()
    out.zero_()
    ext.ffn_gelu(x, wg, wd, hid, out, workspace=ws)
    torch.cuda.synchronize()
    want, want_h = oracle.ffn_gelu(t["x"], t["w1"], t["w2"])
    assert_close(out, want, RTOL, ATOL, "gelu out")
    assert _untouched(hb, F) and _untouched(ob, N)


@pytest.mark.parametrize("S,N,Hq,Hkv,D,P,causal", [
    (150, 256, 4, 2, 128, 40, True),     # many tokens
    (16, 256, 4, 4, 64, 300, False),     # few tokens: split-K projection, key-split attention
])
@pytest.mark.parametrize("variant", ["vanilla", "roco", "keyformer"])
def test_attention_strided(dev, S, N, Hq, Hkv, D, P, causal, variant):
    t = attn_inputs(S, N, Hq, Hkv, D, P=P, w_std=0.06)
    x, xb = _wide(t["x"], dev)
    wq, _ = _wide(t["wq"], dev)
    wk, _ = _wide(t["wk"], dev)
    wv, _ = _wide(t["wv"], dev)
    out, ob = _wide(torch.zeros(S, Hq * D, dtype=torch.float16), dev)
    # caches with padded rows (stride D + 16) and a padded head stride
    L = P + S
    kbuf = torch.full((Hkv, L + 3, D + 16), CANARY, dtype=torch.float16, device=dev)
    vbuf = torch.full((Hkv, L + 3, D + 16), CANARY, dtype=torch.float16, device=dev)
    kc, vc = kbuf[:, :L, :D], vbuf[:, :L, :D]
    kc.copy_(t["k_cache"].to(dev))
    vc.copy_(t["v_cache"].to(dev))
    scale = 1.0 / math.sqrt(D)
    p = ext.attn_params(Hq, Hkv, D, S, kv_prefix=P, scale=scale, causal=causal, tau=1.0, noise_seed=3)
    scratch = scratch_for(p, N, dev)
    kw = dict(n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=scale, causal=causal, kv_prefix=P,
              k_cache=t["k_cache"], v_cache=t["v_cache"])
    if variant == "vanilla":
        ext.qkv_attention(x, None, wq, wk, wv, kc, vc, scratch, None, out, p)
        want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], **kw)
    elif variant == "roco":
        s1b = torch.full((Hq, L + 8), CANARY, dtype=torch.float32, device=dev)
        s2b = torch.full((Hq, L + 8), CANARY, dtype=torch.float32, device=dev)
        s1, s2 = s1b[:, :L], s2b[:, :L]
        ext.roco(x, None, wq, wk, wv, kc, vc, scratch, out, s1, s2, p)
        want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], roco=True, **kw)
        torch.cuda.synchronize()
        assert torch.allclose(s1.cpu(), want["s1"], rtol=2e-3, atol=1e-4)
        assert torch.allclose(s2.cpu(), want["s2"], rtol=2e-3, atol=1e-4)
        assert bool((s1b[:, L:] == CANARY).all()) and bool((s2b[:, L:] == CANARY).all())
    else:
        score = torch.zeros(Hq, L, dtype=torch.float32, device=dev)
        ext.keyformer(x, None, wq, wk, wv, kc, vc, scratch, None, out, score, p)
        want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], keyformer=True, noise_seed=3, tau=1.0, **kw)
        torch.cuda.synchronize()
        assert torch.allclose(score.cpu(), want["score"], rtol=2e-3, atol=1e-4)
    torch.cuda.synchronize()
    assert_close(out, want["O2"], RTOL, ATOL, "O2")
    assert_close(kc[:, P:], want["k_new"], RTOL, ATOL, "appended k rows")
    assert_close(vc[:, P:], want["v_new"], RTOL, ATOL, "appended v rows")
    assert _untouched(ob, Hq * D) and _untouched(xb, N)
    assert bool((kbuf[:, :, D:] == CANARY).all()) and bool((kbuf[:, L:] == CANARY).all())
    assert bool((vbuf[:, :, D:] == CANARY).all()) and bool((vbuf[:, L:] == CANARY).all())
    assert torch.equal(kc[:, :P].cpu(), t["k_cache"][:, :P])
