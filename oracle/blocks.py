"""CPU restatement of the reference's eager baselines (torch, CPU only).

Every function computes in `compute` precision (float32 by default, float64
for the oracle's own self-checks) and rounds to the element type `elem`
(fp16, the reference's type, by default; bf16 for the bf16 kernels) exactly
where the HIP kernels materialise 16-bit tensors in HBM: the normalised
activations of PreNorm, projected q/k/v, the normalised q/k of QKNorm, the
FFN hidden activation, and the final outputs.
"""
import math

import numpy as np
import torch

from .philox import gumbel_noise


def _f(t, compute):
    return t.detach().to(device="cpu", dtype=compute)


def rmsnorm(x, w=None, eps=0.0, compute=torch.float32, out_dtype=torch.float16):
    """y = x * rsqrt(mean(x^2, -1) + eps) [* w].

    Reference: baseline/ref_rms.py:101-102 (w=None, eps=0); the FFN spelling
    x / sqrt(sum(x^2) / N) at baseline/ffn_ref.py:32-35 is the same function.
    """
    xf = _f(x, compute)
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    if w is not None:
        y = y * _f(w, compute)
    return y.to(out_dtype)


def _silu(a):
    # reference spelling FF1b * sigmoid(FF1b), baseline/ffn_ref.py:44
    return a * torch.sigmoid(a)


def ffn_swiglu(x, w_gate, w_up, w_down, compute=torch.float32, elem=torch.float16):
    """out = (silu(x @ w_gate) * (x @ w_up)) @ w_down, hidden rounded to fp16.

    Reference: baseline/ffn_ref.py:37-50 with w_gate = WFF1b, w_up = WFF1a,
    w_down = WFF2.  Returns (out fp16, hidden fp16).
    """
    xf = _f(x, compute)
    g = xf @ _f(w_gate, compute)
    u = xf @ _f(w_up, compute)
    h = (_silu(g) * u).to(elem)
    out = (h.to(compute) @ _f(w_down, compute)).to(elem)
    return out, h


def ffn_gelu(x, w1, w2, compute=torch.float32, elem=torch.float16):
    """out = gelu_erf(x @ w1) @ w2, hidden rounded to fp16.

    Not in the reference (no gelu anywhere in it); defined by the benchmark
    configuration as the Falcon-7B MLP.  Returns (out fp16, hidden fp16).
    """
    xf = _f(x, compute)
    a = xf @ _f(w1, compute)
    h = (0.5 * a * (1.0 + torch.erf(a * (1.0 / math.sqrt(2.0))))).to(elem)
    out = (h.to(compute) @ _f(w2, compute)).to(elem)
    return out, h


def ffn_block(o2, wo, x, wff1a, wff1b, wff2, falcon_tail=False, compute=torch.float32, elem=torch.float16):
    """The reference-shaped FFN block: output projection + residual + RMSNorm
    + SwiGLU + down projection (baseline/ffn_ref.py:24-52); with
    `falcon_tail` the trailing residual + RMSNorm of :114-121.

    Intermediates the kernels write to HBM are rounded to fp16: attn_O2, FF1.
    Returns a dict with attn_O2, FF1, FF2 and (falcon_tail) O_FF_norm.
    """
    n = x.shape[-1]
    attn_o2 = (_f(o2, compute) @ _f(wo, compute) + _f(x, compute)).to(elem)
    a = attn_o2.to(compute)
    norm = a / torch.sqrt(a.pow(2).sum(-1, keepdim=True) / n)
    ff1a = norm @ _f(wff1a, compute)
    ff1b = norm @ _f(wff1b, compute)
    ff1 = (ff1a * _silu(ff1b)).to(elem)
    ff2 = ff1.to(compute) @ _f(wff2, compute)
    out = {"attn_O2": attn_o2, "FF1": ff1, "FF2": ff2.to(elem)}
    if falcon_tail:
        o_ff = ff2 + norm
        out["O_FF_norm"] = (o_ff / torch.sqrt(o_ff.pow(2).sum(-1, keepdim=True) / n)).to(elem)
    return out


def qkv_attention(
    x,
    wq,
    wk,
    wv,
    *,
    n_q_heads,
    n_kv_heads,
    head_dim,
    scale=1.0,
    causal=False,
    kv_prefix=0,
    k_cache=None,
    v_cache=None,
    prenorm=False,
    prenorm_weight=None,
    rms_eps=0.0,
    qknorm=False,
    keyformer=False,
    noise=None,
    noise_seed=None,
    tau=1.0,
    roco=False,
    want_lse=False,
    head_chunk=4,
    noise_head_ids=None,
    compute=torch.float32,
    elem=torch.float16,
    kv_fp8=False,
    k_scale=1.0,
    v_scale=1.0,
    appended_fp8=None,
):
    """QKV projection + (cache append) + softmax attention, all five variants.

    Reference classes (baseline/ref_rms.py): Vanilla :28-82, PreNorm :84-126,
    KeyFormer :128-171, QKNorm :221-265, RoCo :317-357 and their Norm*
    combinations; reference point = scale 1, causal False, n_kv_heads ==
    n_q_heads, eps 0, no norm weight, tau 1.5, noise tensor.

    x [S, N]; wq [N, Hq*D]; wk, wv [N, Hkv*D]; caches [Hkv, >= P+S, D].
    Key j of query i is visible iff (not causal) or j <= P + i.
    KeyFormer perturbed logits: (scale * q.k + g) / tau  (:164 with scale 1).

    Returns dict: O2 fp16 [S, Hq*D]; k_new, v_new fp16 [Hkv, S, D] (the rows
    appended to the caches; k_new is the *normalised* k under QKNorm, :255);
    score fp32 [Hq, P+S] (keyformer); s1, s2 fp32 [Hq, P+S] (roco);
    lse fp32 [Hq, S] (want_lse).
    `noise_head_ids[h]` is the head index fed to the seeded noise generator
    for local head h (used when the oracle is run on a subset of the heads).

    kv_fp8 (no counterpart in the reference, whose caches are fp16): the
    caches are torch.float8_e4m3fn tensors holding value / scale; the new rows
    are appended as fp8(k / k_scale), fp8(v / v_scale) (round to nearest even,
    saturating at +-448) and attention sees scale * fp8 for every key, cached
    or new.  k_new / v_new are then the fp8 rows.  `appended_fp8 = (k_rows,
    v_rows)` replaces the rows this function would append (they are still
    returned as k_new / v_new) by the given fp8 rows for the attention part: a
    single fp16 rounding difference in the projection can land on the other
    side of an fp8 rounding boundary (6 % of the element), so the attention of
    an implementation is checked against the cache contents it produced, and
    those contents separately against k_new / v_new.
    """
    S, N = x.shape
    Hq, Hkv, D, P = n_q_heads, n_kv_heads, head_dim, kv_prefix
    assert Hq % Hkv == 0
    grp = Hq // Hkv
    L = P + S
    xf = _f(x, compute)
    if prenorm:
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + rms_eps)
        if prenorm_weight is not None:
            xf = xf * _f(prenorm_weight, compute)
        xf = xf.to(elem).to(compute)  # X_norm is an fp16 tensor in the reference (:102) and in the kernels
    q = (xf @ _f(wq, compute)).to(elem).view(S, Hq, D).transpose(0, 1)
    k = (xf @ _f(wk, compute)).to(elem).view(S, Hkv, D).transpose(0, 1)
    v = (xf @ _f(wv, compute)).to(elem).view(S, Hkv, D).transpose(0, 1)
    if qknorm:
        qf, kf = q.to(compute), k.to(compute)
        q = (qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + rms_eps)).to(elem)
        k = (kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + rms_eps)).to(elem)
    k_new, v_new = k.contiguous(), v.contiguous()
    if kv_fp8:
        f8 = torch.float8_e4m3fn
        k_new = (k_new.float() / k_scale).clamp(-448.0, 448.0).to(f8)
        v_new = (v_new.float() / v_scale).clamp(-448.0, 448.0).to(f8)
        k_all, v_all = k_new, v_new
        if appended_fp8 is not None:
            k_all, v_all = appended_fp8[0].detach().cpu().view(f8), appended_fp8[1].detach().cpu().view(f8)
        if P > 0:
            k_all = torch.cat([k_cache[:, :P].detach().cpu().view(f8), k_all], dim=1)
            v_all = torch.cat([v_cache[:, :P].detach().cpu().view(f8), v_all], dim=1)
        k_all, v_all = k_all.to(compute) * k_scale, v_all.to(compute) * v_scale
    else:
        if P > 0:
            k_all = torch.cat([k_cache[:, :P].detach().cpu().to(elem), k_new], dim=1)
            v_all = torch.cat([v_cache[:, :P].detach().cpu().to(elem), v_new], dim=1)
        else:
            k_all, v_all = k_new, v_new
        k_all, v_all = k_all.to(compute), v_all.to(compute)

    out = torch.empty(Hq, S, D, dtype=compute)
    res = {"k_new": k_new, "v_new": v_new}
    if keyformer:
        res["score"] = torch.zeros(Hq, L, dtype=torch.float32)
    if roco:
        res["s1"] = torch.zeros(Hq, L, dtype=torch.float32)
        res["s2"] = torch.zeros(Hq, L, dtype=torch.float32)
    if want_lse:
        res["lse"] = torch.zeros(Hq, S, dtype=torch.float32)
    if causal:
        qi = torch.arange(S)[:, None]
        kj = torch.arange(L)[None, :]
        hidden = kj > (P + qi)
    for h0 in range(0, Hq, head_chunk):
        hs = list(range(h0, min(h0 + head_chunk, Hq)))
        kv = [h // grp for h in hs]
        s = torch.matmul(q[hs].to(compute), k_all[kv].transpose(1, 2)) * scale
        if causal:
            s = s.masked_fill(hidden[None], float("-inf"))
        if want_lse:
            res["lse"][hs] = torch.logsumexp(s, dim=-1).float()
        p = torch.softmax(s, dim=-1)
        out[hs] = torch.matmul(p, v_all[kv])
        if roco:
            res["s1"][hs] = p.sum(dim=1).float()
            res["s2"][hs] = p.pow(2).sum(dim=1).float()
        if keyformer:
            if noise is not None:
                g = noise[hs].detach().cpu().to(compute)
            else:
                ids = hs if noise_head_ids is None else [noise_head_ids[h] for h in hs]
                g = torch.from_numpy(np.ascontiguousarray(gumbel_noise(noise_seed, max(ids) + 1, S, L, heads=ids))).to(compute)
            sp = (s + g) / tau
            res["score"][hs] = torch.softmax(sp, dim=-1).sum(dim=1).float()
    res["O2"] = out.transpose(0, 1).reshape(S, Hq * D).to(elem)
    res["q_rows"] = q.transpose(0, 1).reshape(S, Hq * D).contiguous()  # the (normalised) fp16 q the attention used
    return res


def attention_stage(q_rows, k_all, v_all, *, n_q_heads, n_kv_heads, scale=1.0, causal=False, kv_prefix=0,
                    compute=torch.float32, elem=torch.float16):
    """The attention part of `qkv_attention` alone, from given 16-bit q rows [S, Hq*D] and all keys / values
    [Hkv, P+S, D] (baseline/ref_rms.py:60-80: scores, softmax, P.V, heads concatenated).  Used to separate the
    rounding of the projection / normalisation from the attention arithmetic: tests feed it the q, k, v an
    implementation produced.  Pinned by equality with `qkv_attention` on that function's own q, k, v."""
    S = q_rows.shape[0]
    Hq, Hkv = n_q_heads, n_kv_heads
    D = q_rows.shape[1] // Hq
    L = k_all.shape[1]
    assert L == kv_prefix + S
    grp = Hq // Hkv
    q = q_rows.detach().cpu().view(S, Hq, D).transpose(0, 1).to(compute)
    k, v = k_all.detach().cpu().to(compute), v_all.detach().cpu().to(compute)
    out = torch.empty(Hq, S, D, dtype=compute)
    for h in range(Hq):
        s = (q[h] @ k[h // grp].t()) * scale
        if causal:
            s = s.masked_fill(torch.arange(L)[None, :] > (kv_prefix + torch.arange(S)[:, None]), float("-inf"))
        out[h] = torch.softmax(s, dim=-1) @ v[h // grp]
    return out.transpose(0, 1).reshape(S, Hq * D).to(elem)
