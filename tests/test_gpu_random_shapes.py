"""GPU parity on randomly drawn (but seeded, so repeatable) shapes: sequence
lengths, prefixes, head layouts and variant switches that nobody picked by
hand, every case through the C ABI against the CPU oracle.  Tolerances as in
the hand-picked tests: fp16 outputs rtol = atol = 1e-2, fp32 scores 1e-3."""
import math
import random

import pytest
import torch

import oracle
from gpu_util import run_qkv
from test_gpu_attention import assert_scores
from util import assert_close, attn_inputs

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def _draw(seed):
    r = random.Random(seed)
    D = r.choice([64, 128])
    Hkv = r.choice([1, 2, 3])
    Hq = Hkv * r.choice([1, 2, 4])
    few = r.random() < 0.4
    S = r.randint(1, 32) if few else r.randint(33, 300)
    P = r.choice([0, 0, r.randint(1, 700)]) if few else r.choice([0, 0, r.randint(1, 200)])
    N = 8 * r.randint(8, 40)
    causal = r.random() < 0.6
    return S, N, Hq, Hkv, D, P, causal


def _draw_long(seed):
    """Few new tokens against thousands of cached keys: the looping key-split kernel, heads stacked."""
    r = random.Random(seed)
    D = r.choice([64, 128])
    Hkv = r.choice([1, 2, 3])
    Hq = Hkv * r.choice([1, 2, 4, 8])
    S = r.randint(1, 32)
    P = r.randint(2048, 6000)
    N = 8 * r.randint(8, 24)
    causal = r.random() < 0.6
    return S, N, Hq, Hkv, D, P, causal


def _draw_prefill(seed, lo, hi):
    """Several query blocks and key-block pairs: the prefill attention and score kernels proper."""
    r = random.Random(seed)
    D = r.choice([64, 128])
    Hkv = r.choice([1, 2, 4, 8])
    Hq = Hkv * r.choice([1, 2, 4])
    S = r.randint(lo, hi)
    P = r.choice([0, 0, r.randint(1, 400)])
    N = 8 * r.randint(8, 24)
    causal = r.random() < 0.7
    return S, N, Hq, Hkv, D, P, causal


@pytest.mark.parametrize("seed", range(24))
def test_random_shape_all_variants(dev, seed):
    _check_all_variants(dev, seed, _draw(seed))


@pytest.mark.parametrize("seed,lo,hi", [(2000 + i, 129, 900) for i in range(8)] + [(4000 + i, 900, 2600) for i in range(4)] +
                         [(7000 + i, 65, 1400) for i in range(0, 40, 4)])
def test_random_prefill_all_variants(dev, seed, lo, hi):
    _check_all_variants(dev, seed, _draw_prefill(seed, lo, hi))


@pytest.mark.parametrize("seed", range(200, 208))
def test_random_long_prefix_all_variants(dev, seed):
    _check_all_variants(dev, seed, _draw_long(seed))


@pytest.mark.parametrize("group,Hkv,D", [(3, 2, 64), (5, 1, 128), (6, 1, 64), (71, 1, 64)])
def test_long_prefix_group_sizes_not_multiple_of_four(dev, group, Hkv, D):
    """Few tokens against >= 2048 keys with a group size that leaves waves idle in the score kernel's last chunk of
    heads (four heads of a group share a K tile): 3, 5, 6 and Falcon-7B's 71 query heads over one KV head."""
    seed = 300 + group
    r = random.Random(seed)
    cfg = (r.randint(1, 32), 8 * r.randint(8, 24), group * Hkv, Hkv, D, r.randint(2048, 3000), r.random() < 0.5)
    _check_all_variants(dev, seed, cfg)


@pytest.mark.parametrize("cfg", [
    (700, 256, 16, 4, 128, 130, True),    # 16 heads: two per XCD, six query blocks, eleven key-block pairs
    (520, 192, 24, 24, 64, 0, False),     # MHA, three heads per XCD, no mask
    (900, 128, 8, 1, 64, 64, True),       # MQA, one head per XCD, a ragged last query block
    (390, 160, 10, 5, 128, 77, True),     # a head count that is no multiple of eight keeps the plain map
])
def test_prefill_workgroup_maps(dev, cfg):
    """Several query blocks and key-block pairs per head with head counts that are multiples of eight (the prefill
    attention and score kernels then deal the heads to the XCDs in runs of Hq / 8) and one that is not."""
    _check_all_variants(dev, 400 + cfg[0], cfg)


@pytest.mark.parametrize("cfg", [
    (1088, 128, 8, 2, 128, 0, True),     # 17 half blocks of 64 queries: the middle one has no partner
    (1100, 128, 4, 4, 64, 0, True),      # a ragged last half block (12 queries), 64-wide heads
    (700, 160, 8, 1, 128, 512, True),    # behind a cached prefix: every half block sees the 512 keys before it
    (1030, 96, 2, 1, 128, 0, True),      # 17 half blocks, the last of six queries
    (1152, 128, 6, 3, 64, 0, False),     # no mask: nothing to fold, the blocks stay contiguous
    (650, 96, 8, 2, 64, 0, True),        # just past the key count from which eight waves run: 11 half blocks
    (768, 128, 4, 4, 128, 0, True),      # twelve half blocks, six steps
    (1300, 128, 32, 8, 128, 0, True),    # eight query groups: 21 half blocks, the last workgroup holds one
    (1100, 128, 32, 4, 128, 0, True),    # ... 18 half blocks (the last workgroup holds two)
    (1216, 128, 24, 8, 128, 0, True),    # ... 19 half blocks (three)
    (1200, 128, 32, 8, 128, 300, True),  # ... behind a cached prefix
    (2048, 64, 32, 8, 128, 0, True),     # ... a full round of 256 workgroups (the upper end of the range)
    (2048, 64, 32, 32, 64, 0, True),     # 64-wide heads keep the four-wave kernel at this size
])
def test_prefill_folded_half_blocks(dev, cfg):
    """The eight-wave prefill kernels.  At most 256 workgroups and 640 keys or more: two key ways, and under a causal
    mask a late and an early half block of 64 queries per workgroup instead of 128 consecutive queries.  Between
    129 and 256 workgroups of 256 queries under a causal mask: eight query groups - two late and two early half
    blocks - per workgroup."""
    _check_all_variants(dev, 500 + cfg[0], cfg)


@pytest.mark.parametrize("cfg", [
    (1300, 64, 88, 11, 128, 0, True),    # eleven 128-key blocks x 88 heads, a ragged last block and tile
    (900, 64, 96, 8, 64, 200, True),     # behind a cached prefix: nine blocks, the middle one without a partner
    (700, 64, 130, 10, 64, 0, False),    # no mask, a head count that is no multiple of eight
    (1024, 64, 128, 16, 128, 0, True),   # whole blocks and tiles
])
def test_many_heads_short_sequences(dev, cfg):
    """Many heads on short sequences: launches of several hundred workgroups whose key blocks and query tiles are
    few, ragged or unpaired (the score pass pairs key block b with block n - 1 - b)."""
    S = cfg[0]
    _check_all_variants(dev, 600 + S, cfg)


def _check_all_variants(dev, seed, cfg):
    S, N, Hq, Hkv, D, P, causal = cfg
    r = random.Random(1000 + seed)
    prenorm, qknorm = r.random() < 0.4, r.random() < 0.4
    t = attn_inputs(S, N, Hq, Hkv, D, P=P, w_std=0.06)
    scale = 1.0 / math.sqrt(D)
    kw = dict(n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=scale, causal=causal, kv_prefix=P,
              k_cache=t.get("k_cache"), v_cache=t.get("v_cache"))
    what = "S=%d N=%d Hq=%d Hkv=%d D=%d P=%d causal=%s prenorm=%s qknorm=%s" % (S, N, Hq, Hkv, D, P, causal, prenorm,
                                                                                 qknorm)
    print(what, flush=True)
    # plain / PreNorm / QKNorm
    want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], prenorm=prenorm,
                                prenorm_weight=t["norm_w"] if prenorm else None, rms_eps=1e-5, qknorm=qknorm, **kw)
    got = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, P=P, scale=scale, causal=causal, prenorm=prenorm, norm_weight=prenorm,
                  qknorm=qknorm, eps=1e-5)
    assert_close(got["O2"], want["O2"], RTOL, ATOL, "O2 " + what)
    if P:
        assert_close(got["k_cache"][:, P:], want["k_new"], RTOL, ATOL, "k rows " + what)
        assert torch.equal(got["k_cache"][:, :P], t["k_cache"][:, :P])
    # RoCo statistics
    want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], roco=True, **kw)
    got = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, P=P, scale=scale, causal=causal, variant="roco")
    assert_close(got["O2"], want["O2"], RTOL, ATOL, "roco O2 " + what)
    assert_scores(got["s1"], want["s1"], "s1 " + what)
    assert_scores(got["s2"], want["s2"], "s2 " + what)
    # KeyFormer with seeded noise, at the fast temperature and at another one
    for tau in (1.0, 1.5):
        want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], keyformer=True, tau=tau, noise_seed=seed + 5,
                                    **kw)
        got = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, P=P, scale=scale, causal=causal, variant="keyformer", tau=tau,
                      seed=seed + 5)
        assert_close(got["O2"], want["O2"], RTOL, ATOL, "keyformer O2 " + what)
        assert_scores(got["score"], want["score"], "score tau=%g " % tau + what)
    # KeyFormer with a noise tensor (the reference's form)
    noise = torch.randn(Hq, S, P + S, generator=torch.Generator().manual_seed(seed + 9)).half()
    want = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], keyformer=True, tau=1.5, noise=noise, **kw)
    got = run_qkv(t, dev, Hq=Hq, Hkv=Hkv, D=D, P=P, scale=scale, causal=causal, variant="keyformer", tau=1.5,
                  noise=noise)
    assert_close(got["O2"], want["O2"], RTOL, ATOL, "keyformer (noise tensor) O2 " + what)
    assert_scores(got["score"], want["score"], "score (noise tensor) " + what)


def _draw_ffn(seed):
    r = random.Random(seed)
    kind = r.choice(["few", "mid", "many"])
    T = {"few": r.randint(1, 64), "mid": r.randint(65, 300), "many": r.randint(301, 1100)}[kind]
    N = 8 * r.randint(4, 96)
    F = 8 * r.randint(4, 200)
    if r.random() < 0.5:  # multiples of 32 in the reduction dimension open the split-K paths
        N, F = 32 * max(N // 32, 1), 32 * max(F // 32, 1)
    return T, N, F


@pytest.mark.parametrize("seed", range(20))
def test_random_shape_ffn(dev, seed):
    from trinity_amd import ext
    from util import ffn_inputs

    T, N, F = _draw_ffn(seed)
    with_ws = seed % 2 == 0
    print("T=%d N=%d F=%d workspace=%s" % (T, N, F, with_ws), flush=True)
    nbytes = ext.ffn_workspace_bytes(T, N, F) if with_ws else 0
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev) if nbytes else None
    t = ffn_inputs(T, N, F, w_std=0.05)
    want, want_h = oracle.ffn_swiglu(t["x"], t["w1"], t["w_up"], t["w2"])
    hid = torch.zeros(T, F, dtype=torch.float16, device=dev)
    out = torch.zeros(T, N, dtype=torch.float16, device=dev)
    ext.ffn_swiglu(t["x"].to(dev), t["w1"].to(dev), t["w_up"].to(dev), t["w2"].to(dev), hid, out, workspace=ws)
    torch.cuda.synchronize()
    assert_close(hid, want_h, RTOL, ATOL, "swiglu hidden")
    assert_close(out, want, RTOL, ATOL, "swiglu out")
    want, want_h = oracle.ffn_gelu(t["x"], t["w1"], t["w2"])
    hid.zero_()
    out.zero_()
    ext.ffn_gelu(t["x"].to(dev), t["w1"].to(dev), t["w2"].to(dev), hid, out, workspace=ws)
    torch.cuda.synchronize()
    assert_close(hid, want_h, RTOL, ATOL, "gelu hidden")
    assert_close(out, want, RTOL, ATOL, "gelu out")


@pytest.mark.parametrize("seed", range(5000, 5012))
def test_random_shape_ffn_k_contiguous(dev, seed):
    """The same draw with the weights stored K-contiguous (stride[0] == 1), half of the cases with more than a
    thousand rows, half of them with a workspace."""
    from trinity_amd import ext
    from util import ffn_inputs

    r = random.Random(seed)
    T, N, F = _draw_ffn(seed)
    if r.random() < 0.5:
        T = r.randint(1100, 2600)
    N, F = 32 * max(N // 32, 1), 32 * max(F // 32, 1)   # (the layout wants the contracted dimension in 32s)
    with_ws = r.random() < 0.5
    print("T=%d N=%d F=%d workspace=%s" % (T, N, F, with_ws), flush=True)
    nbytes = ext.ffn_workspace_bytes(T, N, F) if with_ws else 0
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev) if nbytes else None
    t = ffn_inputs(T, N, F, w_std=0.05)
    kc = lambda w: w.to(dev).t().contiguous().t()   # (made on the device: a copy to it would be row-major again)
    want, want_h = oracle.ffn_swiglu(t["x"], t["w1"], t["w_up"], t["w2"])
    hid = torch.zeros(T, F, dtype=torch.float16, device=dev)
    out = torch.zeros(T, N, dtype=torch.float16, device=dev)
    ext.ffn_swiglu(t["x"].to(dev), kc(t["w1"]), kc(t["w_up"]), kc(t["w2"]), hid, out, workspace=ws)
    torch.cuda.synchronize()
    assert_close(hid, want_h, RTOL, ATOL, "swiglu hidden")
    assert_close(out, want, RTOL, ATOL, "swiglu out")
    want, want_h = oracle.ffn_gelu(t["x"], t["w1"], t["w2"])
    hid.zero_()
    out.zero_()
    ext.ffn_gelu(t["x"].to(dev), kc(t["w1"]), kc(t["w2"]), hid, out, workspace=ws)
    torch.cuda.synchronize()
    assert_close(hid, want_h, RTOL, ATOL, "gelu hidden")
    assert_close(out, want, RTOL, ATOL, "gelu out")
