"""The C-ABI library loads without a GPU, exports every symbol the header
declares, and rejects bad arguments before anything could be launched."""
import ctypes
import os
import re

import pytest
import torch

from trinity_amd import ext

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_loads_and_exports_header_symbols():
    L = ext.lib()
    header = open(os.path.join(ROOT, "include", "trinity_amd.h")).read()
    declared = set(re.findall(r"\b(tri_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    for name in declared:
        assert hasattr(L, name), "missing export " + name
    assert declared == set(ext.EXPORTS)
    assert L.tri_abi_version() == 8
    assert L.tri_status_string(0) == b"ok"
    assert b"scratch" in L.tri_status_string(-7)


def test_workspace_sizes():
    # few rows: room for fp32 partial sums of every split; many rows: never needed
    assert ext.gemm_workspace_bytes(16, 4096, 12288) > 0
    assert ext.gemm_workspace_bytes(16, 4096, 12288) % (16 * 12288 * 4) == 0
    assert ext.gemm_workspace_bytes(2048, 4096, 14336) == 0        # many rows, a tile count that fills the chip
    assert ext.gemm_workspace_bytes(256, 14336, 4096) > 0          # a handful of tiles over a deep K: split-K
    assert ext.gemm_workspace_bytes(16, 4100, 12288) == 0          # K not a multiple of 32
    assert ext.ffn_workspace_bytes(16, 4096, 14336) >= ext.gemm_workspace_bytes(16, 4096, 2 * 14336)
    assert ext.ffn_workspace_bytes(16, 4096, 14336) >= ext.gemm_workspace_bytes(16, 14336, 4096)
    assert ext.ffn_workspace_bytes(2048, 4096, 14336) == 0
    # the attention scratch grows by the projection's workspace when there are few new tokens
    few = ext.qkv_scratch_bytes(ext.attn_params(32, 32, 128, 16, kv_prefix=1024), 4096)
    assert few >= ext.gemm_workspace_bytes(16, 4096, 3 * 4096)
    x, wg, wu, wd, hid, out = _h(16, 64), _h(64, 128), _h(64, 128), _h(128, 64), _h(16, 128), _h(16, 64)
    ws = torch.zeros(1024, dtype=torch.uint8)
    assert ext.ffn_swiglu(x, wg, wu, wd, hid, out, workspace=ws, validate_only=True) == 0
    assert ext.ffn_swiglu(x, wg, wu, wd, hid, out, workspace=ws.float(), validate_only=True) == -2
    assert ext.ffn_gelu(x, wg, wd, hid, out, workspace=ws.view(2, 512), validate_only=True) == -3


def _h(*shape):
    return torch.zeros(*shape, dtype=torch.float16)


def test_k_contiguous_weights_validation():
    """Weights may be K-contiguous (stride[0] == 1); K must then be a multiple of 32; gate and up share a layout,
    and so do W_q / W_k / W_v."""
    kc = lambda k, n, pad=0: torch.zeros(n, k + pad, dtype=torch.float16)[:, :k].t()
    x, hid, out = _h(16, 64), _h(16, 128), _h(16, 64)
    assert kc(64, 128).stride() == (1, 64)
    assert ext.ffn_swiglu(x, kc(64, 128), kc(64, 128), kc(128, 64), hid, out, validate_only=True) == 0
    assert ext.ffn_swiglu(x, kc(64, 128, 8), kc(64, 128), kc(128, 64, 24), hid, out, validate_only=True) == 0
    assert ext.ffn_swiglu(x, kc(64, 128), _h(64, 128), kc(128, 64), hid, out, validate_only=True) == -4   # mixed gate / up
    assert ext.ffn_swiglu(x, _h(64, 128), _h(64, 128), kc(128, 64), hid, out, validate_only=True) == 0    # down alone
    assert ext.ffn_swiglu(x, kc(64, 128, 4), kc(64, 128, 4), kc(128, 64), hid, out, validate_only=True) == -4
    assert ext.ffn_gelu(x, kc(64, 128), kc(128, 64), hid, out, validate_only=True) == 0
    x2, hid2, out2 = _h(16, 72), _h(16, 128), _h(16, 72)
    assert ext.ffn_gelu(x2, _h(72, 128), _h(128, 72), hid2, out2, validate_only=True) == 0
    assert ext.ffn_gelu(x2, kc(72, 128), _h(128, 72), hid2, out2, validate_only=True) == -6               # K % 32 != 0
    assert ext.ffn_gelu(x, kc(64, 128), kc(64, 64), hid, out, validate_only=True) == -3
    p = ext.attn_params(2, 2, 64, 16, causal=True)
    scratch = torch.zeros(ext.qkv_scratch_bytes(p, 64) + 256, dtype=torch.uint8)
    scratch = scratch[(-scratch.data_ptr()) % 256:][:ext.qkv_scratch_bytes(p, 64)]
    assert ext.qkv_attention(x, None, _h(64, 128), _h(64, 128), _h(64, 128), None, None, scratch, None, _h(16, 128), p,
                             validate_only=True) == 0
    assert ext.qkv_attention(x, None, kc(64, 128), _h(64, 128), _h(64, 128), None, None, scratch, None, _h(16, 128), p,
                             validate_only=True) == -4                                                  # mixed layouts
    assert ext.qkv_attention(x, None, kc(64, 128), kc(64, 128, 8), kc(64, 128), None, None, scratch, None, _h(16, 128), p,
                             validate_only=True) == 0
    x3 = _h(16, 72)
    scratch3 = torch.zeros(ext.qkv_scratch_bytes(p, 72) + 256, dtype=torch.uint8)
    scratch3 = scratch3[(-scratch3.data_ptr()) % 256:][:ext.qkv_scratch_bytes(p, 72)]
    assert ext.qkv_attention(x3, None, _h(72, 128), _h(72, 128), _h(72, 128), None, None, scratch3, None, _h(16, 128), p,
                             validate_only=True) == 0
    assert ext.qkv_attention(x3, None, kc(72, 128), kc(72, 128), kc(72, 128), None, None, scratch3, None, _h(16, 128), p,
                             validate_only=True) == -6                                                  # K % 32 != 0


def test_scratch_size_query_rejects_what_the_launchers_reject():
    """A size is only returned for parameters the entry points accept (a negative return is a status)."""
    q = lambda **kw: ext.lib().tri_qkv_scratch_bytes(ctypes.byref(ext.attn_params(**kw)), ctypes.c_int64(4096))
    ok = dict(n_q_heads=32, n_kv_heads=8, head_dim=128, seq=16, kv_prefix=1024)
    assert q(**ok) > 0
    assert q(**dict(ok, kv_prefix=-5)) == -3
    assert q(**dict(ok, kv_prefix=2 ** 31 - 8)) == -6      # P + S no longer wraps to a plausible size
    assert q(**dict(ok, kv_prefix=2 ** 23)) == -6          # a head's rows exceed a 32-bit buffer descriptor
    assert q(**dict(ok, head_dim=96)) == -6
    assert q(**dict(ok, n_kv_heads=5)) == -3
    assert q(**dict(ok, seq=0)) == -3


def test_static_scratch_entry_point_checks_before_touching_the_gpu():
    """tri_qkv_attention_static refuses a call that does not fit its array, and any bad argument, on the host."""
    S, N, Hq, Hkv, D = 8192, 4096, 32, 8, 128
    x, wq, wkv = _h(S, N), _h(N, Hq * D), _h(N, Hkv * D)
    out = _h(S, Hq * D)
    p = ext.attn_params(Hq, Hkv, D, S, causal=True)
    assert ext.qkv_scratch_bytes(p, N) > ext.STATIC_SCRATCH_BYTES
    assert ext.qkv_attention_static(x, None, wq, wkv, wkv, None, None, None, out, p, status_only=True) == -7
    p16 = ext.attn_params(Hq, Hkv, D, 16, causal=True)
    assert ext.qkv_attention_static(x[:16], None, wq, wkv[:, :8], wkv, None, None, None, out[:16], p16,
                                    status_only=True) == -3
    assert ext.qkv_attention_static(x[:16], None, wq, wkv, wkv, None, None, None, out[:16].float(), p16,
                                    status_only=True) == -2
    header = open(os.path.join(ROOT, "include", "trinity_amd.h")).read()
    assert "#define TRI_STATIC_SCRATCH_BYTES (64 * 1024 * 1024)" in header and ext.STATIC_SCRATCH_BYTES == 64 << 20


@pytest.mark.skipif(torch.cuda.is_available(), reason="a GPU is visible")
def test_prepare_needs_a_device():
    # the list of kernels that want the large-LDS attribute is filled when the library loads; without a GPU the
    # first of them cannot be prepared and the call says so instead of pretending
    assert ext.lib().tri_prepare() == -8


def test_rmsnorm_validation():
    x, y, w = _h(8, 64), _h(8, 64), _h(64)
    assert ext.rmsnorm(x, w, y, validate_only=True) == 0
    assert ext.rmsnorm(x, None, y, validate_only=True) == 0
    assert ext.rmsnorm(x, w, _h(8, 32), validate_only=True) == -3
    assert ext.rmsnorm(x, _h(32), y, validate_only=True) == -3
    assert ext.rmsnorm(x.float(), w, y, validate_only=True) == -2
    assert ext.rmsnorm(x.t(), None, y.t(), validate_only=True) == -4
    assert ext.lib().tri_validate_rmsnorm(None, None, None, ctypes.c_float(0)) == -1


def test_ffn_validation():
    x, wg, wu, wd, hid, out = _h(16, 64), _h(64, 128), _h(64, 128), _h(128, 64), _h(16, 128), _h(16, 64)
    assert ext.ffn_swiglu(x, wg, wu, wd, hid, out, validate_only=True) == 0
    assert ext.ffn_gelu(x, wg, wd, hid, out, validate_only=True) == 0
    assert ext.ffn_swiglu(x, wg, _h(64, 120), wd, hid, out, validate_only=True) == -3
    assert ext.ffn_swiglu(x, wg, wu, wd, _h(16, 64), out, validate_only=True) == -3
    assert ext.ffn_swiglu(x, wg, None, wd, hid, out, validate_only=True) == -1
    assert ext.ffn_gelu(x, wg.t().contiguous().t(), wd, hid, out, validate_only=True) == 0    # K-contiguous weights
    assert ext.ffn_gelu(x.t().contiguous().t(), wg, wd, hid, out, validate_only=True) == -4   # but row-major activations
    assert ext.ffn_gelu(x, wg[:, ::2], _h(64, 64), _h(16, 64), out, validate_only=True) == -4  # neither layout
    assert ext.ffn_gelu(_h(16, 60), _h(60, 128), wd, hid, out, validate_only=True) == -4     # rows not 16-byte multiples
    bad = torch.zeros(16 * 64 + 8, dtype=torch.float16)[4:4 + 16 * 64].view(16, 64)           # 8-byte aligned only
    assert ext.ffn_gelu(bad, wg, wd, hid, out, validate_only=True) == -5
    M, N, Fd = 16, 64, 128
    args = [_h(M, N), _h(N, N), _h(M, N), _h(N, Fd), _h(N, Fd), _h(Fd, N), _h(M, N), torch.zeros(M), _h(M, Fd), _h(M, N)]
    assert ext.ffn_block(*args, validate_only=True) == 0
    assert ext.ffn_block(*args, o_ff_norm=_h(M, N), validate_only=True) == 0
    args[7] = torch.zeros(M - 1)
    assert ext.ffn_block(*args, validate_only=True) == -3


def _qkv_args(S=32, N=64, Hq=4, Hkv=2, D=64, P=0):
    p = ext.attn_params(Hq, Hkv, D, S, kv_prefix=P)
    nbytes = ext.qkv_scratch_bytes(p, N)
    scratch = torch.zeros(nbytes + 256, dtype=torch.uint8)
    off = (-scratch.data_ptr()) % 256
    scratch = scratch[off:off + nbytes]
    t = dict(x=_h(S, N), wq=_h(N, Hq * D), wk=_h(N, Hkv * D), wv=_h(N, Hkv * D), out=_h(S, Hq * D), scratch=scratch, p=p)
    if P:
        t["kc"], t["vc"] = _h(Hkv, P + S, D), _h(Hkv, P + S, D)
    return t


def test_qkv_validation():
    t = _qkv_args()
    v = lambda **o: ext.qkv_attention(o.get("x", t["x"]), o.get("nw"), o.get("wq", t["wq"]), t["wk"], t["wv"],
                                      o.get("kc"), o.get("vc"), o.get("scratch", t["scratch"]), o.get("lse"),
                                      o.get("out", t["out"]), o.get("p", t["p"]), validate_only=True)
    assert v() == 0
    assert v(lse=torch.zeros(4, 32)) == 0
    assert v(lse=torch.zeros(4, 31)) == -3
    assert v(scratch=t["scratch"][:-256]) == -7
    assert v(wq=_h(64, 128)) == -3
    assert v(nw=_h(64)) == -3                      # a norm weight without prenorm
    assert v(p=ext.attn_params(4, 2, 96, 32)) == -6
    assert v(p=ext.attn_params(4, 3, 64, 32)) == -3
    assert v(p=ext.attn_params(4, 2, 64, 1 << 22)) == -6                # projected queries beyond a 32-bit extent
    assert v(p=ext.attn_params(4, 2, 64, 32, kv_prefix=8)) == -1      # prefix without caches
    t2 = _qkv_args(P=8)
    assert ext.qkv_attention(t2["x"], None, t2["wq"], t2["wk"], t2["wv"], t2["kc"], t2["vc"], t2["scratch"], None,
                             t2["out"], t2["p"], validate_only=True) == 0
    assert ext.qkv_attention(t2["x"], None, t2["wq"], t2["wk"], t2["wv"], t2["kc"][:, :30], t2["vc"], t2["scratch"],
                             None, t2["out"], t2["p"], validate_only=True) == -3
    # keyformer / roco extras
    assert ext.keyformer(t["x"], None, t["wq"], t["wk"], t["wv"], None, None, t["scratch"], None, t["out"],
                         torch.zeros(4, 32), t["p"], validate_only=True) == 0
    assert ext.keyformer(t["x"], None, t["wq"], t["wk"], t["wv"], None, None, t["scratch"], _h(4, 32, 32), t["out"],
                         torch.zeros(4, 32), t["p"], validate_only=True) == 0
    assert ext.keyformer(t["x"], None, t["wq"], t["wk"], t["wv"], None, None, t["scratch"], _h(4, 32, 31), t["out"],
                         torch.zeros(4, 32), t["p"], validate_only=True) == -3
    assert ext.roco(t["x"], None, t["wq"], t["wk"], t["wv"], None, None, t["scratch"], t["out"], torch.zeros(4, 32),
                    torch.zeros(4, 32), t["p"], validate_only=True) == 0
    assert ext.roco(t["x"], None, t["wq"], t["wk"], t["wv"], None, None, t["scratch"], t["out"], torch.zeros(4, 32),
                    _h(4, 32), t["p"], validate_only=True) == -2


def test_fp8_cache_validation():
    S, N, Hq, Hkv, D, P = 16, 64, 4, 2, 64, 40
    f8 = torch.float8_e4m3fn
    p = ext.attn_params(Hq, Hkv, D, S, kv_prefix=P, kv_fp8=True, k_scale=0.05, v_scale=0.02)
    nbytes = ext.qkv_scratch_bytes(p, N)
    # room for 16-bit copies of all P + S rows on top of the 16-bit scratch
    assert nbytes >= ext.qkv_scratch_bytes(ext.attn_params(Hq, Hkv, D, S, kv_prefix=P), N) + 2 * Hkv * (P + S) * D * 2
    raw = torch.zeros(nbytes + 256, dtype=torch.uint8)
    off = (-raw.data_ptr()) % 256
    scratch = raw[off:off + nbytes]
    x, wq, wk, wv, out = _h(S, N), _h(N, Hq * D), _h(N, Hkv * D), _h(N, Hkv * D), _h(S, Hq * D)
    kc, vc = torch.zeros(Hkv, P + S, D, dtype=f8), torch.zeros(Hkv, P + S, D, dtype=f8)
    v = lambda kc=kc, vc=vc, p=p, x=x, out=out: ext.qkv_attention(x, None, wq, wk, wv, kc, vc, scratch, None, out, p,
                                                                   validate_only=True)
    assert v() == 0
    assert v(kc=_h(Hkv, P + S, D), vc=_h(Hkv, P + S, D)) == -2          # 16-bit caches with kv_fp8 set
    assert v(kc=None, vc=None) == -1                                     # fp8 mode needs its caches, also at P = 0
    assert v(p=ext.attn_params(Hq, Hkv, D, S, kv_prefix=P)) == -2        # fp8 caches without kv_fp8
    assert v(p=ext.attn_params(Hq, Hkv, D, S, kv_prefix=P, kv_fp8=True, k_scale=0.0, v_scale=1.0)) == -6
    assert v(kc=torch.zeros(Hkv, P + S - 1, D, dtype=f8)) == -3
    assert v(kc=torch.zeros(Hkv, P + S, D + 8, dtype=f8)[:, :, :D]) == -4   # rows of 72 bytes: not 16-byte multiples
    xb = x.bfloat16()
    assert ext.qkv_attention(xb, None, wq.bfloat16(), wk.bfloat16(), wv.bfloat16(), kc, vc, scratch, None,
                             out.bfloat16(), p, validate_only=True) == 0   # bf16 activations, fp8 caches


def test_no_silent_fallback_when_library_missing(monkeypatch):
    monkeypatch.setattr(ext, "_lib", None)
    monkeypatch.setattr(ext, "LIB_PATH", "/nonexistent/libtrinity_amd.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        ext.lib()


def test_empty_batch_is_legal():
    """No token rows: every FFN / RMSNorm entry point validates (and, on a GPU, launches nothing)."""
    e = torch.zeros(0, 64, dtype=torch.float16)
    assert ext.rmsnorm(e, _h(64), torch.zeros(0, 64, dtype=torch.float16), validate_only=True) == 0
    assert ext.ffn_swiglu(e, _h(64, 128), _h(64, 128), _h(128, 64), torch.zeros(0, 128, dtype=torch.float16),
                          torch.zeros(0, 64, dtype=torch.float16), validate_only=True) == 0
    assert ext.ffn_gelu(e, _h(64, 128), _h(128, 64), torch.zeros(0, 128, dtype=torch.float16),
                        torch.zeros(0, 64, dtype=torch.float16), validate_only=True) == 0
    # the reference-shaped block too: its fp32 row buffer has no elements then and may have no storage
    z = lambda *sh: torch.zeros(*sh, dtype=torch.float16)
    assert ext.ffn_block(e, _h(64, 64), z(0, 64), _h(64, 128), _h(64, 128), _h(128, 64), z(0, 64),
                         torch.zeros(0, dtype=torch.float32), z(0, 128), z(0, 64), validate_only=True) == 0
    # but a missing weight matrix is still an error
    assert ext.ffn_gelu(e, None, _h(128, 64), torch.zeros(0, 128, dtype=torch.float16),
                        torch.zeros(0, 64, dtype=torch.float16), validate_only=True) == -1


def test_mixed_element_types_are_rejected():
    """A call is fp16 or bf16 throughout (the element type of its first activation tensor)."""
    BF = torch.bfloat16
    x = torch.zeros(16, 64, dtype=BF)
    w = torch.zeros(64, 128, dtype=torch.float16)
    assert ext.ffn_gelu(x, w, torch.zeros(128, 64, dtype=BF), torch.zeros(16, 128, dtype=BF),
                        torch.zeros(16, 64, dtype=BF), validate_only=True) == -2
    assert ext.rmsnorm(x, torch.zeros(64, dtype=torch.float16), torch.zeros(16, 64, dtype=BF), validate_only=True) == -2
    assert ext.ffn_gelu(x, w.to(BF), torch.zeros(128, 64, dtype=BF), torch.zeros(16, 128, dtype=BF),
                        torch.zeros(16, 64, dtype=BF), validate_only=True) == 0
    assert ext.rmsnorm(torch.zeros(16, 64), None, torch.zeros(16, 64), validate_only=True) == -2       # fp32 elements


# ---------------------------------------------------------------- randomised validation
# The validators must give a defined status for any combination of shapes, strides and element types, and accept
# every consistent one; nothing here launches a kernel.
from hypothesis import given, settings, strategies as st  # noqa: E402

_DT = [torch.float16, torch.bfloat16, torch.float32]


@settings(max_examples=150, deadline=None)
@given(m=st.integers(0, 40), n=st.sampled_from([8, 60, 64, 72, 200, 4096]), dn=st.sampled_from([0, 0, 0, 8, -8]),
       dt=st.sampled_from(_DT), wdt=st.sampled_from(_DT), with_w=st.booleans(), transpose=st.booleans())
def test_rmsnorm_validation_randomised(m, n, dn, dt, wdt, with_w, transpose):
    x = torch.zeros(m, n, dtype=dt)
    y = torch.zeros(m, max(n + dn, 8), dtype=dt)
    w = torch.zeros(n, dtype=wdt) if with_w else None
    if transpose and m > 0:
        x, y = x.t(), y.t()
    rc = ext.rmsnorm(x, w, y, validate_only=True)
    assert -8 <= rc <= 0
    consistent = dn == 0 and dt != torch.float32 and (w is None or wdt == dt) and not (transpose and m > 0) \
        and n % 8 == 0
    if consistent:
        assert rc == 0
    if dt == torch.float32:
        assert rc != 0


@settings(max_examples=150, deadline=None)
@given(m=st.integers(0, 70), n=st.sampled_from([64, 128, 96]), f=st.sampled_from([64, 128, 256]),
       df=st.sampled_from([0, 0, 0, 8]), dt=st.sampled_from(_DT[:2]), wdt=st.sampled_from(_DT[:2]),
       ws_bytes=st.sampled_from([None, 0, 256, 1 << 20]))
def test_ffn_validation_randomised(m, n, f, df, dt, wdt, ws_bytes):
    x, hid, out = torch.zeros(m, n, dtype=dt), torch.zeros(m, f, dtype=dt), torch.zeros(m, n, dtype=dt)
    wg, wu, wd = torch.zeros(n, f, dtype=wdt), torch.zeros(n, f + df, dtype=wdt), torch.zeros(f, n, dtype=wdt)
    ws = None if ws_bytes is None else torch.zeros(ws_bytes, dtype=torch.uint8)
    rc = ext.ffn_swiglu(x, wg, wu, wd, hid, out, workspace=ws, validate_only=True)
    assert -8 <= rc <= 0
    if df == 0 and dt == wdt:
        assert rc == 0          # a workspace of any size is legal: too small a one only disables the split path
    if dt != wdt:
        assert rc in (-2, -3) and (rc == -2 or df != 0)
    elif df != 0:
        assert rc == -3
    rc2 = ext.ffn_gelu(x, wg, wd, hid, out, workspace=ws, validate_only=True)
    assert rc2 == (0 if dt == wdt else -2)


@settings(max_examples=150, deadline=None)
@given(s=st.integers(0, 48), hq=st.sampled_from([1, 4, 6, 8]), group=st.sampled_from([1, 2, 4, 3]),
       d=st.sampled_from([64, 128, 96, 32]), p=st.sampled_from([0, 0, 8, 33]), causal=st.booleans(),
       short_scratch=st.booleans(), dt=st.sampled_from(_DT[:2]))
def test_qkv_validation_randomised(s, hq, group, d, p, causal, short_scratch, dt):
    hkv = max(hq // group, 1)
    n = 64
    prm = ext.attn_params(hq, hkv, d, s, kv_prefix=p, causal=causal)
    x = torch.zeros(s, n, dtype=dt)
    wq, wk, wv = (torch.zeros(n, hq * d, dtype=dt), torch.zeros(n, hkv * d, dtype=dt), torch.zeros(n, hkv * d, dtype=dt))
    kc = vc = None
    if p > 0:
        kc, vc = torch.zeros(hkv, p + s, d, dtype=dt), torch.zeros(hkv, p + s, d, dtype=dt)
    if s == 0:  # attention wants at least one new token
        with pytest.raises(ext.TrinityError):
            ext.qkv_scratch_bytes(prm, n)
        return
    good_shape = d in (64, 128) and hq % hkv == 0
    nbytes = ext.qkv_scratch_bytes(prm, n) if good_shape else 1 << 20
    assert nbytes >= 0
    raw = torch.zeros(max(nbytes - (256 if short_scratch else 0), 0) + 256, dtype=torch.uint8)
    lead = (-raw.data_ptr()) % 256  # the scratch buffer has to be 256-byte aligned
    scratch = raw[lead:lead + raw.numel() - 256]
    out = torch.zeros(s, hq * d, dtype=dt)
    rc = ext.qkv_attention(x, None, wq, wk, wv, kc, vc, scratch, None, out, prm, validate_only=True)
    assert -8 <= rc <= 0
    if d not in (64, 128):
        assert rc == -6
    elif hq % hkv != 0:
        assert rc == -3
    elif short_scratch and nbytes >= 256:
        assert rc == -7
    else:
        assert rc == 0


def test_header_is_plain_c_and_links(tmp_path):
    """include/trinity_amd.h compiles as C99 with warnings as errors, and a C program linked against the library
    reaches the entry points (no GPU work: version, status strings, a validator, a size query)."""
    import shutil
    import subprocess

    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    src = tmp_path / "use.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include "trinity_amd.h"
int main(void) {
  tri_tensor x;
  tri_attn_params p;
  memset(&x, 0, sizeof x);
  memset(&p, 0, sizeof p);
  if (tri_abi_version() != TRI_ABI_VERSION) return 1;
  if (strcmp(tri_status_string(TRI_OK), "ok") != 0) return 2;
  if (tri_validate_rmsnorm(NULL, NULL, NULL, 0.0f) != TRI_ERR_NULL) return 3;
  x.ndim = 2; x.shape[0] = 4; x.shape[1] = 64; x.stride[0] = 64; x.stride[1] = 1; x.dtype = TRI_F16;
  if (tri_validate_rmsnorm(&x, NULL, &x, 0.0f) != TRI_ERR_NULL) return 4;   /* no storage behind the rows */
  p.n_q_heads = 4; p.n_kv_heads = 2; p.head_dim = 64; p.seq = 16; p.scale = 0.125f; p.tau = 1.0f;
  if (tri_qkv_scratch_bytes(&p, 256) <= 0) return 5;
  if (tri_gemm_workspace_bytes(16, 4096, 12288) <= 0) return 6;
  printf("abi %d ok\n", tri_abi_version());
  return 0;
}
''')
    exe = tmp_path / "use"
    libdir = os.path.dirname(ext.LIB_PATH)
    cmd = ["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), str(src),
           "-o", str(exe), "-L", libdir, "-ltrinity_amd", "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, "exit %d: %s %s" % (r.returncode, r.stdout, r.stderr)
    assert "ok" in r.stdout
