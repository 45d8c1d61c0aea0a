"""Pins for the CPU oracle (no GPU): each function is checked against an
independent library routine, a closed form or a brute-force loop, chosen so
that a dropped term, a wrong sign/index or a transposed operand fails."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle.philox import philox4x32, philox4x32_10, uniform_from_bits, gumbel_noise
from util import attn_inputs, ffn_inputs, gen, randn


# ----------------------------------------------------------------- Philox / Gumbel
def test_philox_known_answers():
    # Random123 kat_vectors, philox4x32 with 10 rounds
    kat = [
        ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
        ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
        ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
         (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
    ]
    for ctr, key, want in kat:
        got = tuple(int(x) for x in philox4x32_10(*ctr, *key))
        assert got == want
    # the same file's vectors for seven rounds - the round count of the kernels' noise
    kat7 = [
        ((0, 0, 0, 0), (0, 0), (0x5F6FB709, 0x0D893F64, 0x4F121F81, 0x4F730A48)),
        ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x5207DDC2, 0x45165E59, 0x4D8EE751, 0x8C52F662)),
        ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
         (0x4DFCCABA, 0x190A87F0, 0xC47362BA, 0xB6B5242A)),
    ]
    for ctr, key, want in kat7:
        assert tuple(int(x) for x in philox4x32(*ctr, *key, rounds=7)) == want
        assert tuple(int(x) for x in philox4x32(*ctr, *key)) == want   # the default is the kernels' count


def test_uniform_open_interval_and_fp32_exact():
    x = np.array([0, 1, 0x1FF, 0x200, 0xFFFF], dtype=np.uint32)
    u = uniform_from_bits(x)
    assert (u > 0).all() and (u < 1).all()
    assert (u.astype(np.float32).astype(np.float64) == u).all()
    assert u[0] == 2.0 ** -17 and u[-1] == 1 - 2.0 ** -17


def test_gumbel_moments_and_layout():
    g = gumbel_noise(7, 2, 64, 1000)
    assert g.shape == (2, 64, 1000) and g.dtype == np.float32
    assert abs(g.mean() - 0.5772) < 0.02          # Euler-Mascheroni
    assert abs(g.var() - math.pi ** 2 / 6) < 0.05
    # head restriction and key truncation select the same numbers
    g1 = gumbel_noise(7, 2, 64, 1000, heads=[1])
    assert np.array_equal(g1[0], g[1])
    assert np.array_equal(gumbel_noise(7, 2, 64, 10)[:, :, :10], g[:, :, :10])
    # element (h, q, k): counter (2 * (k // 16) + (k // 4) % 2, q, h, 0), word k % 4, low half of the word when
    # (k // 8) % 2 == 0, else the high half.  k = 37: call 2 * 2 + 1 = 5, word 1, low half; k = 45: same call,
    # same word, high half.
    w = philox4x32(np.uint32(5), np.uint32(5), np.uint32(1), np.uint32(0), np.uint32(7), np.uint32(0))
    for k, bits in ((37, int(w[1]) & 0xFFFF), (45, int(w[1]) >> 16)):
        u = (bits + 0.5) / 65536.0
        assert g[1, 5, k] == np.float32(-np.log(-np.log(u)))
    # every key of a row draws from its own sixteen bits: no two keys of a call share a half word
    from oracle.philox import noise_bits
    calls = {}
    for k in range(64):
        calls.setdefault((2 * (k // 16) + (k // 4) % 2), []).append((k % 4, (k // 8) % 2))
    assert all(len(v) == 8 and len(set(v)) == 8 for v in calls.values())
    b = noise_bits(7, 1, 4, 4096)
    assert b.max() <= 0xFFFF and abs(b.mean() / 65535.0 - 0.5) < 0.02
    # adjacent keys and the two halves of a word are uncorrelated
    c1 = np.corrcoef(b[0, 0, :-1].astype(np.float64), b[0, 0, 1:].astype(np.float64))[0, 1]
    c8 = np.corrcoef(b[0, 0, :-8].astype(np.float64), b[0, 0, 8:].astype(np.float64))[0, 1]
    assert abs(c1) < 0.06 and abs(c8) < 0.06


# ----------------------------------------------------------------- RMSNorm
def test_rmsnorm_matches_torch_rms_norm():
    g = gen(1)
    x = randn(g, 33, 200)
    w = randn(g, 200, std=0.1, mean=1.0)
    want = F.rms_norm(x.double(), (200,), w.double(), eps=1e-5)
    got = oracle.rmsnorm(x, w, 1e-5, compute=torch.float64, out_dtype=torch.float64)
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)
    # reference point: no weight, no eps (baseline/ref_rms.py:101-102)
    want0 = x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True))
    assert torch.allclose(oracle.rmsnorm(x, None, 0.0, compute=torch.float64, out_dtype=torch.float64), want0)


def test_rmsnorm_closed_forms():
    w = torch.linspace(0.5, 1.5, 64)
    x = torch.full((3, 64), -2.5)
    y = oracle.rmsnorm(x, w, 0.0, compute=torch.float64, out_dtype=torch.float64)
    assert torch.allclose(y, -w.double().expand(3, 64))        # constant row -> sign(c) * w
    g = gen(2)
    x = randn(g, 5, 64)
    a = oracle.rmsnorm(x, None, 0.0, compute=torch.float64, out_dtype=torch.float64)
    b = oracle.rmsnorm(x * 4, None, 0.0, compute=torch.float64, out_dtype=torch.float64)
    assert torch.allclose(a, b)                                 # scale invariance at eps = 0
    assert torch.allclose(a.pow(2).mean(-1), torch.ones(5, dtype=torch.float64))


# ----------------------------------------------------------------- FFN
def test_ffn_swiglu_against_library_ops():
    t = ffn_inputs(24, 64, 96, gated=True, w_std=0.2)
    out, hid = oracle.ffn_swiglu(t["x"], t["w1"], t["w_up"], t["w2"], compute=torch.float64)
    x = t["x"].double()
    h = (F.silu(x @ t["w1"].double()) * (x @ t["w_up"].double())).half()
    assert torch.equal(hid, h)
    assert torch.equal(out, (h.double() @ t["w2"].double()).half())
    # swapping gate and up must change the result (guards against a transposed pair)
    out2, _ = oracle.ffn_swiglu(t["x"], t["w_up"], t["w1"], t["w2"], compute=torch.float64)
    assert not torch.equal(out, out2)


def test_ffn_gelu_against_library_ops():
    t = ffn_inputs(24, 64, 96, gated=False, w_std=0.2)
    out, hid = oracle.ffn_gelu(t["x"], t["w1"], t["w2"], compute=torch.float64)
    h = F.gelu(t["x"].double() @ t["w1"].double(), approximate="none").half()
    assert torch.equal(hid, h)
    assert torch.equal(out, (h.double() @ t["w2"].double()).half())


def test_ffn_block_composition():
    g = gen(3)
    M, N, Fd = 16, 64, 96
    o2, x = randn(g, M, N, std=0.5), randn(g, M, N, std=0.5)
    wo, a, b, w2 = randn(g, N, N, std=0.1), randn(g, N, Fd, std=0.1), randn(g, N, Fd, std=0.1), randn(g, Fd, N, std=0.1)
    r = oracle.ffn_block(o2, wo, x, a, b, w2, falcon_tail=True, compute=torch.float64)
    attn = (o2.double() @ wo.double() + x.double()).half()
    assert torch.equal(r["attn_O2"], attn)
    norm = F.rms_norm(attn.double(), (N,), None, eps=0.0)
    ff1 = ((norm @ a.double()) * F.silu(norm @ b.double())).half()
    assert torch.equal(r["FF1"], ff1)
    ff2 = ff1.double() @ w2.double()
    assert torch.equal(r["FF2"], ff2.half())
    assert torch.equal(r["O_FF_norm"], F.rms_norm(ff2 + norm, (N,), None, eps=0.0).half())


# ----------------------------------------------------------------- attention
def _sdpa(q, k, v, causal, scale, P):
    # q [Hq,S,D], k/v [Hkv,L,D] float64
    Hq, S, D = q.shape
    grp = Hq // k.shape[0]
    k = k.repeat_interleave(grp, dim=0)
    v = v.repeat_interleave(grp, dim=0)
    L = k.shape[1]
    mask = None
    if causal:
        mask = torch.arange(L)[None, :] <= (P + torch.arange(S))[:, None]
    return F.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=scale)


@pytest.mark.parametrize("causal,P,Hq,Hkv", [(True, 0, 4, 2), (False, 0, 4, 4), (False, 24, 4, 1), (True, 24, 6, 2)])
def test_attention_against_sdpa(causal, P, Hq, Hkv):
    S, N, D = 40, 64, 16
    t = attn_inputs(S, N, Hq, Hkv, D, P=P, w_std=0.2)
    scale = 0.37
    r = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=scale,
                             causal=causal, kv_prefix=P, k_cache=t.get("k_cache"), v_cache=t.get("v_cache"),
                             compute=torch.float64, head_chunk=3)
    x = t["x"].double()
    q = (x @ t["wq"].double()).half().view(S, Hq, D).transpose(0, 1).double()
    k = (x @ t["wk"].double()).half().view(S, Hkv, D).transpose(0, 1)
    v = (x @ t["wv"].double()).half().view(S, Hkv, D).transpose(0, 1)
    assert torch.equal(r["k_new"], k.contiguous()) and torch.equal(r["v_new"], v.contiguous())
    if P:
        k = torch.cat([t["k_cache"][:, :P], k], 1)
        v = torch.cat([t["v_cache"][:, :P], v], 1)
    want = _sdpa(q, k.double(), v.double(), causal, scale, P).transpose(0, 1).reshape(S, Hq * D)
    assert torch.allclose(r["O2"].double(), want, rtol=0, atol=2e-3)
    assert (r["O2"].double() - want).abs().max() < 1.1 * want.abs().max() * 2 ** -11 + 1e-6   # only the final rounding


@pytest.mark.parametrize("causal,qknorm", [(True, False), (False, True), (True, True)])
def test_attention_stage_equals_the_whole_block(causal, qknorm):
    """attention_stage on the q rows / keys / values qkv_attention itself used reproduces its O2 bit for bit
    (grouped heads, cached prefix, with and without the mask and QKNorm)."""
    S, N, D, Hq, Hkv, P = 9, 32, 8, 4, 2, 5
    t = attn_inputs(S, N, Hq, Hkv, D, P=P, w_std=0.3)
    kw = dict(n_q_heads=Hq, n_kv_heads=Hkv, scale=0.7, causal=causal, kv_prefix=P)
    r = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], head_dim=D, k_cache=t["k_cache"], v_cache=t["v_cache"],
                             qknorm=qknorm, rms_eps=1e-6, **kw)
    k_all = torch.cat([t["k_cache"][:, :P], r["k_new"]], dim=1)
    v_all = torch.cat([t["v_cache"][:, :P], r["v_new"]], dim=1)
    assert torch.equal(oracle.attention_stage(r["q_rows"], k_all, v_all, **kw), r["O2"])
    # and it does depend on what it is given
    assert not torch.equal(oracle.attention_stage(r["q_rows"] * 2, k_all, v_all, **kw), r["O2"])


def test_attention_brute_force_tiny():
    S, N, D, Hq, Hkv, P = 5, 8, 4, 2, 1, 3
    t = attn_inputs(S, N, Hq, Hkv, D, P=P, w_std=0.5)
    r = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=0.5,
                             causal=True, kv_prefix=P, k_cache=t["k_cache"], v_cache=t["v_cache"], roco=True,
                             want_lse=True, compute=torch.float64)
    x = t["x"].double()
    q = (x @ t["wq"].double()).half().double()
    k = (x @ t["wk"].double()).half().double()
    v = (x @ t["wv"].double()).half().double()
    O = torch.zeros(S, Hq * D, dtype=torch.float64)
    s1 = torch.zeros(Hq, P + S, dtype=torch.float64)
    s2 = torch.zeros(Hq, P + S, dtype=torch.float64)
    for h in range(Hq):
        for i in range(S):
            logits = []
            for j in range(P + i + 1):
                kj = t["k_cache"][0, j].double() if j < P else k[j - P, 0:D]
                logits.append(0.5 * float((q[i, h * D:(h + 1) * D] * kj).sum()))
            mx = max(logits)
            e = [math.exp(l - mx) for l in logits]
            z = sum(e)
            assert abs(float(r["lse"][h, i]) - (mx + math.log(z))) < 1e-5
            for j, ej in enumerate(e):
                vj = t["v_cache"][0, j].double() if j < P else v[j - P, 0:D]
                O[i, h * D:(h + 1) * D] += ej / z * vj
                s1[h, j] += ej / z
                s2[h, j] += (ej / z) ** 2
    assert torch.allclose(r["O2"].double(), O, rtol=0, atol=2e-3)
    assert torch.allclose(r["s1"].double(), s1, rtol=1e-6, atol=1e-7)
    assert torch.allclose(r["s2"].double(), s2, rtol=1e-6, atol=1e-7)


def test_attention_invariants():
    S, N, D, Hq, Hkv = 32, 32, 8, 4, 2
    t = attn_inputs(S, N, Hq, Hkv, D, w_std=0.3)
    kw = dict(n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=0.3, compute=torch.float64)
    r = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], causal=True, roco=True, keyformer=True, noise_seed=3,
                             tau=1.3, **kw)
    assert torch.allclose(r["s1"].sum(-1).double(), torch.full((Hq,), float(S), dtype=torch.float64), atol=1e-4)
    assert torch.allclose(r["score"].sum(-1).double(), torch.full((Hq,), float(S), dtype=torch.float64), atol=1e-4)
    assert (r["s2"] <= r["s1"] + 1e-7).all()
    # zero noise, tau 1: the KeyFormer score is RoCo's s1
    z = torch.zeros(Hq, S, S, dtype=torch.float16)
    r0 = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], causal=True, roco=True, keyformer=True, noise=z,
                              tau=1.0, **kw)
    assert torch.allclose(r0["score"], r0["s1"], rtol=1e-6, atol=1e-7)
    # non-causal: permuting the tokens permutes the rows of O2 and the per-key sums
    perm = torch.randperm(S, generator=gen(9))
    a = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], causal=False, roco=True, **kw)
    b = oracle.qkv_attention(t["x"][perm], t["wq"], t["wk"], t["wv"], causal=False, roco=True, **kw)
    assert torch.allclose(a["O2"][perm].double(), b["O2"].double(), atol=1e-3)
    assert torch.allclose(a["s1"][:, perm], b["s1"], rtol=1e-5, atol=1e-6)


def _keyformer_brute_force(t, g, *, S, Hq, Hkv, D, P, scale, tau, causal):
    """score[h, j] = sum_i exp((scale * q_i.k_j + g[h,i,j]) / tau) / sum_j' exp((scale * q_i.k_j' + g[h,i,j']) / tau),
    over the keys visible to query i, with explicit loops (baseline/ref_rms.py:163-166 with scale 1, tau 1.5;
    keyformer_falcon_benchmark4358.py:122-141: C_out = sum over the queries of exp(C_perturb) / C_sum_perturb)."""
    x = t["x"].double()
    q = (x @ t["wq"].double()).half().double()
    k = (x @ t["wk"].double()).half().double()
    grp = Hq // Hkv
    score = torch.zeros(Hq, P + S, dtype=torch.float64)
    for h in range(Hq):
        hk = h // grp
        for i in range(S):
            last = P + i if causal else P + S - 1
            e = []
            for j in range(last + 1):
                kj = t["k_cache"][hk, j].double() if j < P else k[j - P, hk * D:(hk + 1) * D]
                logit = scale * float((q[i, h * D:(h + 1) * D] * kj).sum())
                e.append(math.exp((logit + float(g[h, i, j])) / tau))
            z = sum(e)
            for j, ej in enumerate(e):
                score[h, j] += ej / z
    return score


@pytest.mark.parametrize("causal", [False, True])
def test_keyformer_score_brute_force_tiny(causal):
    # noise tensor, tau = 1.5 (the reference's point), a cached prefix, grouped heads; logits of order 1 and noise of
    # order 1 so that a dropped noise term, s / tau + g or a sum over the wrong axis all move the result
    S, N, D, Hq, Hkv, P = 5, 8, 4, 4, 2, 3
    t = attn_inputs(S, N, Hq, Hkv, D, P=P, w_std=0.5)
    g = randn(gen(11), Hq, S, P + S, std=1.0)
    r = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=0.7,
                             causal=causal, kv_prefix=P, k_cache=t["k_cache"], v_cache=t["v_cache"], keyformer=True,
                             noise=g, tau=1.5, compute=torch.float64)
    want = _keyformer_brute_force(t, g.double(), S=S, Hq=Hq, Hkv=Hkv, D=D, P=P, scale=0.7, tau=1.5, causal=causal)
    assert torch.allclose(r["score"].double(), want, rtol=1e-6, atol=1e-7)
    # the pin is sharp: the same loops with the two nearest wrong formulas are far away
    for wrong in (lambda l, n: l / 1.5 + n, lambda l, n: l / 1.5):
        x = t["x"].double()
        q = (x @ t["wq"].double()).half().double().view(S, Hq, D)
        kn = (x @ t["wk"].double()).half().double().view(S, Hkv, D).transpose(0, 1)
        ka = torch.cat([t["k_cache"][:, :P].double(), kn], 1)
        lg = 0.7 * torch.einsum("ihd,hjd->hij", q, ka.repeat_interleave(Hq // Hkv, 0))
        sp = wrong(lg, g.double())
        if causal:
            sp = sp.masked_fill(torch.arange(P + S)[None, :] > P + torch.arange(S)[:, None], float("-inf"))
        assert (torch.softmax(sp, -1).sum(1) - want).abs().max() > 1e-2


@pytest.mark.parametrize("seeded", [False, True])
def test_keyformer_score_zero_logits_closed_form(seeded):
    # wq = 0: every logit is 0, so score = softmax(g / tau) over the keys, summed over the queries - computed here
    # with the library softmax on the noise alone, for a noise tensor and for the seeded generator
    S, N, D, Hq, Hkv, P, tau = 12, 16, 8, 2, 1, 4, 1.5
    t = attn_inputs(S, N, Hq, Hkv, D, P=P)
    t["wq"].zero_()
    L = P + S
    if seeded:
        g = torch.from_numpy(gumbel_noise(5, Hq, S, L)).double()
        kw = dict(noise_seed=5)
    else:
        gt = randn(gen(4), Hq, S, L, std=2.0)
        g, kw = gt.double(), dict(noise=gt)
    for causal in (False, True):
        r = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=1.0,
                                 causal=causal, kv_prefix=P, k_cache=t["k_cache"], v_cache=t["v_cache"], keyformer=True,
                                 tau=tau, compute=torch.float64, **kw)
        z = g / tau
        if causal:
            z = z.masked_fill(torch.arange(L)[None, :] > P + torch.arange(S)[:, None], float("-inf"))
        want = F.softmax(z, dim=-1).sum(dim=1)
        assert torch.allclose(r["score"].double(), want, rtol=1e-6, atol=1e-7)


def test_keyformer_score_depends_on_tau_and_noise():
    S, N, D, Hq, Hkv = 16, 16, 8, 2, 2
    t = attn_inputs(S, N, Hq, Hkv, D, w_std=0.4)
    g = randn(gen(6), Hq, S, S, std=1.0)
    kw = dict(n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=0.5, causal=True, keyformer=True, compute=torch.float64)
    a = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], noise=g, tau=1.0, **kw)["score"]
    b = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], noise=g, tau=1.5, **kw)["score"]
    c = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], noise=torch.zeros_like(g), tau=1.5, **kw)["score"]
    assert (a - b).abs().max() > 1e-2 and (b - c).abs().max() > 1e-2
    # tau scales logits and noise alike: doubling tau, the softmax scale and the noise leaves the score unchanged
    d = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], noise=(g.float() * 2).half(), tau=3.0,
                             **dict(kw, scale=1.0))["score"]
    assert torch.allclose(b, d, rtol=1e-5, atol=1e-6)


def test_roco_uniform_attention_closed_forms():
    # wq = 0 -> all logits 0 -> uniform attention
    S, N, D, Hq, Hkv, P = 16, 16, 8, 2, 2, 4
    t = attn_inputs(S, N, Hq, Hkv, D, P=P)
    t["wq"].zero_()
    kw = dict(n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=1.0, kv_prefix=P, k_cache=t["k_cache"], v_cache=t["v_cache"],
              roco=True, compute=torch.float64)
    r = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], causal=False, **kw)
    L = P + S
    assert torch.allclose(r["s1"].double(), torch.full((Hq, L), S / L, dtype=torch.float64), rtol=1e-6)
    assert torch.allclose(r["s2"].double(), torch.full((Hq, L), S / L ** 2, dtype=torch.float64), rtol=1e-6)
    r = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], causal=True, **kw)
    want1 = torch.tensor([sum(1.0 / (P + i + 1) for i in range(S) if j <= P + i) for j in range(L)], dtype=torch.float64)
    want2 = torch.tensor([sum(1.0 / (P + i + 1) ** 2 for i in range(S) if j <= P + i) for j in range(L)], dtype=torch.float64)
    assert torch.allclose(r["s1"].double(), want1.expand(Hq, L), rtol=1e-6)
    assert torch.allclose(r["s2"].double(), want2.expand(Hq, L), rtol=1e-6)


def test_prenorm_and_qknorm_paths():
    S, N, D, Hq, Hkv = 24, 32, 8, 4, 1
    t = attn_inputs(S, N, Hq, Hkv, D, w_std=0.3)
    kw = dict(n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=0.5, causal=True, compute=torch.float64)
    # PreNorm == Vanilla on pre-normalised input (fp64 input keeps the comparison exact up to rounding of q/k/v)
    xn = F.rms_norm(t["x"].double(), (N,), t["norm_w"].double(), eps=1e-5).half()   # X_norm is materialised in fp16
    a = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], prenorm=True, prenorm_weight=t["norm_w"], rms_eps=1e-5, **kw)
    b = oracle.qkv_attention(xn, t["wq"], t["wk"], t["wv"], **kw)
    assert torch.equal(a["O2"], b["O2"])
    # QKNorm: the appended keys have unit RMS per head row, and O2 is invariant to scaling wq / wk
    c = oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], qknorm=True, **kw)
    assert torch.allclose(c["k_new"].double().pow(2).mean(-1), torch.ones(Hkv, S, dtype=torch.float64), atol=2e-3)
    d = oracle.qkv_attention(t["x"], (t["wq"].float() * 2).half(), (t["wk"].float() * 0.5).half(), t["wv"], qknorm=True, **kw)
    assert torch.allclose(c["O2"].double(), d["O2"].double(), atol=2e-3)
    assert not torch.allclose(c["O2"].double(), oracle.qkv_attention(t["x"], t["wq"], t["wk"], t["wv"], **kw)["O2"].double(), atol=2e-3)


# ----------------------------------------------------------------- fp8 KV caches
def test_fp8_cache_definition():
    """scale * fp8 for every key; with a scale that makes the quantisation exact the result equals the fp16-cache
    one, and the appended rows saturate at +-448 instead of turning into NaN."""
    import math as _m
    from oracle import qkv_attention
    g = gen(3)
    S, N, Hq, Hkv, D, P = 6, 32, 2, 1, 64, 5
    x, wq = randn(g, S, N), randn(g, N, Hq * D, std=0.1)
    # weights with entries in {-1, 0, 1} / 8 and inputs in {-1, 0, 1}: k, v are multiples of 1/8 below 448 / 8
    x = torch.randint(-1, 2, (S, N), generator=g).half()
    wk = (torch.randint(-1, 2, (N, Hkv * D), generator=g).float() / 8).half()
    wv = (torch.randint(-1, 2, (N, Hkv * D), generator=g).float() / 8).half()
    kc16 = (torch.randint(-8, 9, (Hkv, P + S, D), generator=g).float() / 8).half()
    vc16 = (torch.randint(-8, 9, (Hkv, P + S, D), generator=g).float() / 8).half()
    kw = dict(n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, scale=1 / _m.sqrt(D), causal=True, kv_prefix=P)
    ref = qkv_attention(x, wq, wk, wv, k_cache=kc16, v_cache=vc16, **kw)
    assert (ref["k_new"].float().abs() <= 4).all()   # |k| <= 32 / 8: exact in e4m3 after division by 1 / 8
    f8 = torch.float8_e4m3fn
    got = qkv_attention(x, wq, wk, wv, k_cache=(kc16.float() * 8).to(f8), v_cache=(vc16.float() * 8).to(f8),
                        kv_fp8=True, k_scale=0.125, v_scale=0.125, **kw)
    assert torch.equal(got["O2"], ref["O2"])
    assert torch.equal(got["k_new"].float() * 0.125, ref["k_new"].float())
    # saturation
    big = qkv_attention(x, wq, wk * 64, wv, k_cache=(kc16.float() * 8).to(f8), v_cache=(vc16.float() * 8).to(f8),
                        kv_fp8=True, k_scale=1e-3, v_scale=0.125, **kw)
    assert torch.isfinite(big["k_new"].float()).all() and big["k_new"].float().abs().max() == 448
