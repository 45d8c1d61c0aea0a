"""Seeded inputs shared by the parity tests (generated on the CPU so that the
oracle and the device see identical bits; seed convention of the reference's
driver, convert_eval_rms.py:127)."""

import torch


def gen(seed=42):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def randn(g, *shape, std=1.0, mean=0.0):
    return (torch.randn(*shape, generator=g) * std + mean).to(torch.float16)


def attn_inputs(S, N, Hq, Hkv, D, P=0, seed=42, x_std=1.0, w_std=0.02, cache_std=1.0, with_cache=None):
    g = gen(seed)
    t = {
        "x": randn(g, S, N, std=x_std),
        "wq": randn(g, N, Hq * D, std=w_std),
        "wk": randn(g, N, Hkv * D, std=w_std),
        "wv": randn(g, N, Hkv * D, std=w_std),
        "norm_w": randn(g, N, std=0.1, mean=1.0),
    }
    if with_cache is None:
        with_cache = P > 0
    if with_cache:
        t["k_cache"] = randn(g, Hkv, P + S, D, std=cache_std)
        t["v_cache"] = randn(g, Hkv, P + S, D, std=cache_std)
    return t


def ffn_inputs(T, N, F, N2=None, seed=42, x_std=1.0, w_std=0.02, gated=True):
    g = gen(seed)
    N2 = N if N2 is None else N2
    t = {"x": randn(g, T, N, std=x_std), "w1": randn(g, N, F, std=w_std)}
    if gated:
        t["w_up"] = randn(g, N, F, std=w_std)
    t["w2"] = randn(g, F, N2, std=w_std)
    return t


def rel_err(a, b, floor=1e-6):
    a = a.double().cpu()
    b = b.double().cpu()
    return ((a - b).abs() / b.abs().clamp_min(floor)).max().item()


def assert_close(actual, expected, rtol, atol, what=""):
    a = actual.double().cpu()
    e = expected.double().cpu()
    assert a.shape == e.shape, (what, a.shape, e.shape)
    assert torch.isfinite(a).all(), what + ": non-finite values"
    err = (a - e).abs()
    tol = atol + rtol * e.abs()
    bad = err > tol
    if bad.any():
        idx = torch.nonzero(bad)[0].tolist()
        raise AssertionError(
            "%s: %d / %d elements out of tolerance (rtol %g, atol %g); max abs err %g; first bad index %s: got %g want %g"
            % (what, int(bad.sum()), a.numel(), rtol, atol, err.max().item(), idx, a[tuple(idx)].item(), e[tuple(idx)].item())
        )
