"""GPU parity (through the C ABI) of RMSNorm and the FFN blocks against the
CPU oracle.  Tolerances: fp16 outputs rtol = atol = 1e-2 (the stated bar)."""
import math

import pytest
import torch

import oracle
from trinity_amd import ext
from util import assert_close, ffn_inputs, gen, randn

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


@pytest.mark.parametrize("rows,n,weight,eps", [
    (4096, 4096, True, 1e-5),      # the benchmark configuration
    (16, 4544, False, 0.0),        # the reference's point (M = 16, Falcon width, no weight, no eps)
    (37, 4544, True, 1e-5),
    (1, 8, True, 1e-5),
    (5, 8192, True, 1e-6),
    (3, 10240, True, 1e-5),        # longer than the register-resident path
    (7, 100, False, 1e-5),         # not a multiple of 8
])
def test_rmsnorm_parity(dev, rows, n, weight, eps):
    g = gen(42)
    x = randn(g, rows, n)
    w = randn(g, n, std=0.1, mean=1.0) if weight else None
    want = oracle.rmsnorm(x, w, eps)
    y = torch.zeros(rows, n, dtype=torch.float16, device=dev)
    ext.rmsnorm(x.to(dev), w.to(dev) if weight else None, y, eps)
    torch.cuda.synchronize()
    # one fp16 rounding of an fp32 product on both sides: essentially exact
    assert_close(y, want, 2e-3, 1e-3, "rmsnorm %dx%d" % (rows, n))


def test_rmsnorm_strided_rows_and_properties(dev):
    g = gen(1)
    big = randn(g, 64, 4096 + 64).to(dev)
    x = big[:, :4096]                      # row stride 4160
    y = torch.zeros(64, 4096, dtype=torch.float16, device=dev)
    ext.rmsnorm(x, None, y, 0.0)
    y2 = torch.zeros_like(y)
    ext.rmsnorm((x.float() * 4).half(), None, y2, 0.0)
    torch.cuda.synchronize()
    assert_close(y, oracle.rmsnorm(x.cpu(), None, 0.0), 2e-3, 1e-3, "strided")
    assert_close(y2, y, 2e-3, 2e-3, "scale invariance")
    assert torch.allclose(y.float().pow(2).mean(-1).cpu(), torch.ones(64), atol=2e-3)


@pytest.mark.parametrize("T,N,F,N2", [
    (300, 512, 1088, 512),      # ragged token count, F not a multiple of the tile
    (256, 256, 256, 256),
    (64, 4544, 1024, 4544),     # Falcon width (71 * 64)
    (1, 64, 64, 64),
])
def test_ffn_swiglu_parity(dev, T, N, F, N2):
    t = ffn_inputs(T, N, F, N2, w_std=0.05)
    want, want_h = oracle.ffn_swiglu(t["x"], t["w1"], t["w_up"], t["w2"])
    hid = torch.zeros(T, F, dtype=torch.float16, device=dev)
    out = torch.zeros(T, N2, dtype=torch.float16, device=dev)
    ext.ffn_swiglu(t["x"].to(dev), t["w1"].to(dev), t["w_up"].to(dev), t["w2"].to(dev), hid, out)
    torch.cuda.synchronize()
    assert_close(hid, want_h, RTOL, ATOL, "swiglu hidden")
    assert_close(out, want, RTOL, ATOL, "swiglu out")


@pytest.mark.parametrize("T,N,F", [(300, 512, 1088), (128, 4544, 2048)])
def test_ffn_gelu_parity(dev, T, N, F):
    t = ffn_inputs(T, N, F, gated=False, w_std=0.05)
    want, want_h = oracle.ffn_gelu(t["x"], t["w1"], t["w2"])
    hid = torch.zeros(T, F, dtype=torch.float16, device=dev)
    out = torch.zeros(T, N, dtype=torch.float16, device=dev)
    ext.ffn_gelu(t["x"].to(dev), t["w1"].to(dev), t["w2"].to(dev), hid, out)
    torch.cuda.synchronize()
    assert_close(hid, want_h, RTOL, ATOL, "gelu hidden")
    assert_close(out, want, RTOL, ATOL, "gelu out")


def _kc(w, pad=0):
    """The same [K, N] matrix stored K-contiguous (the transpose view of a row-major [N, K (+ pad)] tensor)."""
    K, N = w.shape
    store = torch.zeros(N, K + pad, dtype=w.dtype, device=w.device)
    store[:, :K] = w.t()
    return store[:, :K].t()


@pytest.mark.parametrize("T,N,F,N2,pad", [
    (300, 512, 1088, 512, 0),      # ragged token count, column counts that end inside a tile
    (256, 256, 256, 256, 8),       # padded weight rows (column stride 264)
    (64, 4544, 1024, 4544, 0),     # few rows: this layout still takes the large tiles
    (1, 64, 64, 64, 0),
    (513, 1024, 544, 264, 0),      # K = 544 = 17 k tiles for the down projection
])
def test_ffn_swiglu_k_contiguous_weights(dev, T, N, F, N2, pad):
    """W_gate / W_up / W_down given K-contiguous (stride[0] == 1): same results as the row-major call."""
    t = ffn_inputs(T, N, F, N2, w_std=0.05)
    want, want_h = oracle.ffn_swiglu(t["x"], t["w1"], t["w_up"], t["w2"])
    hid = torch.zeros(T, F, dtype=torch.float16, device=dev)
    out = torch.zeros(T, N2, dtype=torch.float16, device=dev)
    wg, wu, wd = (_kc(t[k].to(dev), pad) for k in ("w1", "w_up", "w2"))
    assert wg.stride(0) == 1 and wg.shape == (N, F)
    ext.ffn_swiglu(t["x"].to(dev), wg, wu, wd, hid, out)
    torch.cuda.synchronize()
    assert_close(hid, want_h, RTOL, ATOL, "swiglu hidden, K-contiguous weights")
    assert_close(out, want, RTOL, ATOL, "swiglu out, K-contiguous weights")
    # mixed: K-contiguous gate / up, row-major down projection, through the two half entry points
    hid2 = torch.zeros_like(hid)
    out2 = torch.zeros_like(out)
    ext.gateup_swiglu(t["x"].to(dev), wg, wu, None, hid2)
    ext.matmul(hid2, t["w2"].to(dev), None, out2)
    torch.cuda.synchronize()
    assert torch.equal(hid2, hid)
    assert_close(out2, want, RTOL, ATOL, "row-major down projection after K-contiguous gate/up")


@pytest.mark.parametrize("T,N,F", [(300, 512, 1088), (128, 4544, 2048)])
def test_ffn_gelu_k_contiguous_weights(dev, T, N, F):
    t = ffn_inputs(T, N, F, gated=False, w_std=0.05)
    want, want_h = oracle.ffn_gelu(t["x"], t["w1"], t["w2"])
    hid = torch.zeros(T, F, dtype=torch.float16, device=dev)
    out = torch.zeros(T, N, dtype=torch.float16, device=dev)
    ext.ffn_gelu(t["x"].to(dev), _kc(t["w1"].to(dev)), _kc(t["w2"].to(dev)), hid, out)
    torch.cuda.synchronize()
    assert_close(hid, want_h, RTOL, ATOL, "gelu hidden, K-contiguous weights")
    assert_close(out, want, RTOL, ATOL, "gelu out, K-contiguous weights")


def test_matmul_k_contiguous_weight_with_residual(dev):
    g = gen(8)
    M, K, N = 200, 384, 776
    x, w, r = randn(g, M, K), randn(g, K, N, std=0.05), randn(g, M, N)
    out = torch.zeros(M, N, dtype=torch.float16, device=dev)
    ext.matmul(x.to(dev), _kc(w.to(dev)), r.to(dev), out)
    torch.cuda.synchronize()
    want = (x.float() @ w.float() + r.float()).half()
    assert_close(out, want, RTOL, ATOL, "x.w + residual, K-contiguous w")


def test_ffn_swiglu_llama_full_size_k_contiguous(dev):
    """The benchmark shape with the weights stored K-contiguous; the oracle checks a row sample, and the row-major
    call on the same values must agree everywhere (both accumulate each output in the same k order)."""
    T, N, F = 2048, 4096, 14336
    t = ffn_inputs(T, N, F)
    d = {k: v.to(dev) for k, v in t.items()}
    hid = torch.zeros(T, F, dtype=torch.float16, device=dev)
    out = torch.zeros(T, N, dtype=torch.float16, device=dev)
    ext.ffn_swiglu(d["x"], _kc(d["w1"]), _kc(d["w_up"]), _kc(d["w2"]), hid, out)
    hid_r = torch.zeros_like(hid)
    out_r = torch.zeros_like(out)
    ext.ffn_swiglu(d["x"], d["w1"], d["w_up"], d["w2"], hid_r, out_r)
    torch.cuda.synchronize()
    rows = _rows_subset(T, 32, 7)
    want, want_h = oracle.ffn_swiglu(t["x"][rows], t["w1"], t["w_up"], t["w2"])
    assert_close(hid.cpu()[rows], want_h, RTOL, ATOL, "llama hidden, K-contiguous weights")
    assert_close(out.cpu()[rows], want, RTOL, ATOL, "llama out, K-contiguous weights")
    assert_close(hid, hid_r, 1e-3, 1e-3, "hidden: K-contiguous against row-major weights")
    assert_close(out, out_r, 2e-3, 2e-3, "out: K-contiguous against row-major weights")


def _rows_subset(T, k, seed):
    return torch.randperm(T, generator=gen(seed))[:k].sort().values


def test_ffn_swiglu_llama_full_size_row_sample(dev):
    """The benchmark shape; rows are independent, so the oracle checks a sample."""
    T, N, F = 2048, 4096, 14336
    t = ffn_inputs(T, N, F)
    hid = torch.zeros(T, F, dtype=torch.float16, device=dev)
    out = torch.zeros(T, N, dtype=torch.float16, device=dev)
    ext.ffn_swiglu(t["x"].to(dev), t["w1"].to(dev), t["w_up"].to(dev), t["w2"].to(dev), hid, out)
    torch.cuda.synchronize()
    rows = _rows_subset(T, 48, 5)
    want, want_h = oracle.ffn_swiglu(t["x"][rows], t["w1"], t["w_up"], t["w2"])
    assert_close(hid.cpu()[rows], want_h, RTOL, ATOL, "llama hidden")
    assert_close(out.cpu()[rows], want, RTOL, ATOL, "llama out")
    # linearity of the down projection in the hidden activation: out(2h) = 2 out(h) needs no oracle
    assert torch.isfinite(out).all()


def test_ffn_gelu_falcon_full_size_row_sample(dev):
    T, N, F = 2048, 4544, 18176
    t = ffn_inputs(T, N, F, gated=False)
    hid = torch.zeros(T, F, dtype=torch.float16, device=dev)
    out = torch.zeros(T, N, dtype=torch.float16, device=dev)
    ext.ffn_gelu(t["x"].to(dev), t["w1"].to(dev), t["w2"].to(dev), hid, out)
    torch.cuda.synchronize()
    rows = _rows_subset(T, 48, 6)
    want, want_h = oracle.ffn_gelu(t["x"][rows], t["w1"], t["w2"])
    assert_close(hid.cpu()[rows], want_h, RTOL, ATOL, "falcon hidden")
    assert_close(out.cpu()[rows], want, RTOL, ATOL, "falcon out")


@pytest.mark.parametrize("M,N,F,falcon", [(16, 512, 1024, False), (16, 4544, 512, True), (40, 256, 320, True)])
def test_ffn_block_reference_shape(dev, M, N, F, falcon):
    """The reference's own FFN block (M = 16 tokens, inputs scaled as in convert_ffn_llama.py:86-96)."""
    g = gen(42)
    sc = 0.05
    o2, x = randn(g, M, N, std=sc), randn(g, M, N, std=sc)
    wo, a, b, w2 = randn(g, N, N, std=sc), randn(g, N, F, std=sc), randn(g, N, F, std=sc), randn(g, F, N, std=sc)
    want = oracle.ffn_block(o2, wo, x, a, b, w2, falcon_tail=falcon)
    d = lambda v: v.to(dev)
    attn = torch.zeros(M, N, dtype=torch.float16, device=dev)
    rs = torch.zeros(M, dtype=torch.float32, device=dev)
    ff1 = torch.zeros(M, F, dtype=torch.float16, device=dev)
    ff2 = torch.zeros(M, N, dtype=torch.float16, device=dev)
    onorm = torch.zeros(M, N, dtype=torch.float16, device=dev) if falcon else None
    ext.ffn_block(d(o2), d(wo), d(x), d(a), d(b), d(w2), attn, rs, ff1, ff2, onorm)
    torch.cuda.synchronize()
    assert_close(attn, want["attn_O2"], RTOL, ATOL, "attn_O2")
    assert_close(ff1, want["FF1"], RTOL, ATOL, "FF1")
    assert_close(ff2, want["FF2"], RTOL, ATOL, "FF2")
    if falcon:
        assert_close(onorm, want["O_FF_norm"], RTOL, ATOL, "O_FF_norm")


def _ws(dev, nbytes):
    return torch.zeros(max(nbytes, 16), dtype=torch.uint8, device=dev)


@pytest.mark.parametrize("T,N,F,N2", [
    (16, 512, 1088, 512),       # the reference's token count; F not a multiple of the 128-column slab
    (1, 64, 64, 64),
    (33, 4544, 1024, 4544),     # Falcon width, second row tile partly filled
    (64, 256, 2048, 256),       # the largest few-row case
])
def test_ffn_few_rows_split_k_parity(dev, T, N, F, N2):
    """With a workspace the few-row (split-K) kernels run; they must agree with the oracle and with the
    large-tile kernels (no workspace)."""
    t = ffn_inputs(T, N, F, N2, w_std=0.05)
    d = {k: v.to(dev) for k, v in t.items()}
    nbytes = ext.ffn_workspace_bytes(T, N, F)
    assert nbytes > 0
    ws = _ws(dev, nbytes)
    for act in ("swiglu", "gelu"):
        hid, out = (torch.zeros(T, F, dtype=torch.float16, device=dev), torch.zeros(T, N2, dtype=torch.float16, device=dev))
        hid0, out0 = torch.zeros_like(hid), torch.zeros_like(out)
        if act == "swiglu":
            want, want_h = oracle.ffn_swiglu(t["x"], t["w1"], t["w_up"], t["w2"])
            ext.ffn_swiglu(d["x"], d["w1"], d["w_up"], d["w2"], hid, out, workspace=ws)
            ext.ffn_swiglu(d["x"], d["w1"], d["w_up"], d["w2"], hid0, out0)
        else:
            want, want_h = oracle.ffn_gelu(t["x"], t["w1"], t["w2"])
            ext.ffn_gelu(d["x"], d["w1"], d["w2"], hid, out, workspace=ws)
            ext.ffn_gelu(d["x"], d["w1"], d["w2"], hid0, out0)
        torch.cuda.synchronize()
        assert_close(hid, want_h, RTOL, ATOL, act + " hidden")
        assert_close(out, want, RTOL, ATOL, act + " out")
        assert_close(hid, hid0.cpu(), 2e-3, 2e-3, act + " hidden vs large tiles")
    # a workspace that is too small silently selects the large-tile kernels
    small = _ws(dev, 64)
    out1 = torch.zeros(T, N2, dtype=torch.float16, device=dev)
    ext.ffn_gelu(d["x"], d["w1"], d["w2"], hid, out1, workspace=small)
    torch.cuda.synchronize()
    assert_close(out1, want, RTOL, ATOL, "gelu out, small workspace")


def test_matmul_residual_and_rowscale_few_rows(dev):
    g = gen(9)
    M, K, N = 16, 1024, 768
    x, w, r = randn(g, M, K), randn(g, K, N, std=0.05), randn(g, M, N)
    rs = (torch.rand(M, generator=g) + 0.5).float()
    ws = _ws(dev, ext.gemm_workspace_bytes(M, K, 2 * N))
    out = torch.zeros(M, N, dtype=torch.float16, device=dev)
    ext.matmul(x.to(dev), w.to(dev), r.to(dev), out, workspace=ws)
    torch.cuda.synchronize()
    assert_close(out, (x.float() @ w.float() + r.float()).half(), RTOL, ATOL, "x.w + residual")
    w2 = randn(g, K, N, std=0.05)
    hid = torch.zeros(M, N, dtype=torch.float16, device=dev)
    ext.gateup_swiglu(x.to(dev), w.to(dev), w2.to(dev), rs.to(dev), hid, workspace=ws)
    torch.cuda.synchronize()
    a, b = (x.float() @ w.float()) * rs[:, None], (x.float() @ w2.float()) * rs[:, None]
    assert_close(hid, (a * torch.sigmoid(a) * b).half(), RTOL, ATOL, "row-scaled swiglu")


def test_ffn_block_reference_full_shape_with_workspace(dev):
    """The reference's Llama FFN block at its own size (M = 16, N = 4096, P = 14336;
    evaluation/ffn/ffn_llama/tensor_configs.json), inputs as convert_ffn_llama.py:86-96 scales them."""
    M, N, F = 16, 4096, 14336
    g = gen(42)
    sc = 0.02
    o2, x = randn(g, M, N, std=sc), randn(g, M, N, std=sc)
    wo, a, b, w2 = randn(g, N, N, std=sc), randn(g, N, F, std=sc), randn(g, N, F, std=sc), randn(g, F, N, std=sc)
    want = oracle.ffn_block(o2, wo, x, a, b, w2)
    d = lambda v: v.to(dev)
    attn = torch.zeros(M, N, dtype=torch.float16, device=dev)
    rs = torch.zeros(M, dtype=torch.float32, device=dev)
    ff1 = torch.zeros(M, F, dtype=torch.float16, device=dev)
    ff2 = torch.zeros(M, N, dtype=torch.float16, device=dev)
    ws = _ws(dev, ext.ffn_workspace_bytes(M, N, F))
    ext.ffn_block(d(o2), d(wo), d(x), d(a), d(b), d(w2), attn, rs, ff1, ff2, None, workspace=ws)
    torch.cuda.synchronize()
    assert_close(attn, want["attn_O2"], RTOL, ATOL, "attn_O2")
    assert_close(ff1, want["FF1"], RTOL, ATOL, "FF1")
    assert_close(ff2, want["FF2"], RTOL, ATOL, "FF2")


def test_activation_functions_pointwise(dev):
    """GELU and SiLU of the epilogues on a dense grid of arguments: identity weights make the hidden
    activation gelu(x) / silu(x) element by element; both must round to the fp16 value of the fp64 function
    (one fp16 ulp of slack)."""
    T, N = 512, 64
    grid = torch.linspace(-9.0, 9.0, T * (N - 1), dtype=torch.float64).reshape(T, N - 1)
    x = torch.cat([grid, torch.ones(T, 1, dtype=torch.float64)], dim=1).half()      # last column: constant 1
    eye = torch.eye(N, dtype=torch.float16)
    gate = eye.clone(); gate[N - 1, N - 1] = 0
    up = torch.zeros(N, N, dtype=torch.float16); up[N - 1, :] = 1                      # x . up = 1 everywhere
    hid = torch.zeros(T, N, dtype=torch.float16, device=dev)
    out = torch.zeros(T, N, dtype=torch.float16, device=dev)
    xd = x.to(dev)
    a = x.double()[:, : N - 1]
    for ws in (None, _ws(dev, ext.ffn_workspace_bytes(T, N, N))):                     # T > 64: both use the large tiles
        ext.ffn_gelu(xd, eye.to(dev), eye.to(dev), hid, out, workspace=ws)
        torch.cuda.synchronize()
        want = (0.5 * a * (1 + torch.erf(a / math.sqrt(2.0)))).half()
        got = hid.cpu()[:, : N - 1]
        ulp = torch.maximum(want.abs().float() * 2 ** -10, torch.tensor(2.0 ** -24))
        assert ((got.float() - want.float()).abs() <= ulp).all(), "gelu"
        ext.ffn_swiglu(xd, gate.to(dev), up.to(dev), eye.to(dev), hid, out, workspace=ws)
        torch.cuda.synchronize()
        want = (a * torch.sigmoid(a)).half()
        got = hid.cpu()[:, : N - 1]
        ulp = torch.maximum(want.abs().float() * 2 ** -10, torch.tensor(2.0 ** -24))
        assert ((got.float() - want.float()).abs() <= ulp).all(), "silu"
    # the few-row kernels share the functions
    ws = _ws(dev, ext.ffn_workspace_bytes(16, N, N))
    ext.ffn_gelu(xd[:16], eye.to(dev), eye.to(dev), hid[:16], out[:16], workspace=ws)
    torch.cuda.synchronize()
    a16 = a[:16]
    want = (0.5 * a16 * (1 + torch.erf(a16 / math.sqrt(2.0)))).half()
    assert ((hid.cpu()[:16, : N - 1].float() - want.float()).abs() <= torch.maximum(want.abs().float() * 2 ** -10, torch.tensor(2.0 ** -24))).all()


def test_large_split_k_ragged_shape_with_residual(dev):
    """Split-K of a many-row product: ragged M and N, residual added in the merge."""
    g = gen(11)
    M, K, N = 300, 4096, 1288
    nbytes = ext.gemm_workspace_bytes(M, K, N)
    assert nbytes > 0, "this shape is expected to take the split-K plan"
    x, w, r = randn(g, M, K, std=0.5), randn(g, K, N, std=0.03), randn(g, M, N)
    out = torch.zeros(M, N, dtype=torch.float16, device=dev)
    ext.matmul(x.to(dev), w.to(dev), r.to(dev), out, workspace=_ws(dev, nbytes))
    torch.cuda.synchronize()
    assert_close(out, (x.float() @ w.float() + r.float()).half(), RTOL, ATOL, "split-K x.w + residual")


@pytest.mark.parametrize("M,K,N", [
    (2048, 1024, 4544),   # 256 x 160 tiles (17.75 column tiles of 256 fill the chip badly)
    (2048, 512, 6144),    # 256 x 192 tiles
    (1024, 512, 6144),    # 256 x 96 tiles
    (2048, 512, 18176),   # full rounds of 256 x 256 tiles plus a narrower remainder
    (1000, 512, 4672),    # ragged rows and a ragged last column tile
])
def test_matmul_tile_plan_family(dev, M, K, N):
    """Shapes that make the launcher pick each second tile shape of its plan family."""
    g = gen(13)
    x, w = randn(g, M, K, std=0.5), randn(g, K, N, std=0.05)
    out = torch.zeros(M, N, dtype=torch.float16, device=dev)
    ext.matmul(x.to(dev), w.to(dev), None, out)
    torch.cuda.synchronize()
    assert_close(out, (x.float() @ w.float()).half(), RTOL, ATOL, "x.w")


def test_empty_batch_launches_nothing(dev):
    """Zero token rows through the real entry points: status ok, nothing written, no fault."""
    N, F = 64, 128
    e = torch.zeros(0, N, dtype=torch.float16, device=dev)
    w = torch.ones(N, dtype=torch.float16, device=dev)
    ext.rmsnorm(e, w, torch.zeros(0, N, dtype=torch.float16, device=dev), 1e-5)
    wg, wu, wd = (torch.ones(N, F, dtype=torch.float16, device=dev), torch.ones(N, F, dtype=torch.float16, device=dev),
                  torch.ones(F, N, dtype=torch.float16, device=dev))
    ext.ffn_swiglu(e, wg, wu, wd, torch.zeros(0, F, dtype=torch.float16, device=dev), torch.zeros(0, N, dtype=torch.float16, device=dev))
    ext.ffn_gelu(e, wg, wd, torch.zeros(0, F, dtype=torch.float16, device=dev), torch.zeros(0, N, dtype=torch.float16, device=dev))
    torch.cuda.synchronize()
