"""Device-side drivers for the parity tests: move seeded CPU tensors to the
GPU, call the C ABI through trinity_amd.ext, return CPU results."""
import torch

from trinity_amd import ext


def scratch_for(params, n_model, dev):
    return torch.empty(ext.qkv_scratch_bytes(params, n_model), dtype=torch.uint8, device=dev)


def run_qkv(t, dev, *, Hq, Hkv, D, P=0, scale=None, causal=True, prenorm=False, norm_weight=True, qknorm=False,
            eps=0.0, variant="vanilla", noise=None, seed=0, tau=1.0, want_lse=False, mean_var=False,
            keep_scratch=False):
    S, N = t["x"].shape
    p = ext.attn_params(Hq, Hkv, D, S, kv_prefix=P, scale=scale, causal=causal, rms_eps=eps, prenorm=prenorm,
                        qknorm=qknorm, tau=tau, noise_seed=seed)
    d = {k: v.to(dev) for k, v in t.items()}
    kc, vc = d.get("k_cache"), d.get("v_cache")
    nw = d["norm_w"] if (prenorm and norm_weight) else None
    out = torch.zeros(S, Hq * D, dtype=torch.float16, device=dev)
    scratch = scratch_for(p, N, dev)
    res = {}
    if variant == "vanilla":
        lse = torch.zeros(Hq, S, dtype=torch.float32, device=dev) if want_lse else None
        ext.qkv_attention(d["x"], nw, d["wq"], d["wk"], d["wv"], kc, vc, scratch, lse, out, p)
        if want_lse:
            res["lse"] = lse.cpu()
    elif variant == "keyformer":
        score = torch.zeros(Hq, P + S, dtype=torch.float32, device=dev)
        nz = noise.to(dev) if noise is not None else None
        ext.keyformer(d["x"], nw, d["wq"], d["wk"], d["wv"], kc, vc, scratch, nz, out, score, p)
        res["score"] = score.cpu()
    elif variant == "roco":
        s1 = torch.zeros(Hq, P + S, dtype=torch.float32, device=dev)
        s2 = torch.zeros(Hq, P + S, dtype=torch.float32, device=dev)
        ext.roco(d["x"], nw, d["wq"], d["wk"], d["wv"], kc, vc, scratch, out, s1, s2, p, as_mean_var=mean_var)
        res["s1"], res["s2"] = s1.cpu(), s2.cpu()
    else:
        raise ValueError(variant)
    torch.cuda.synchronize()
    res["O2"] = out.cpu()
    if keep_scratch:
        res["scratch"] = scratch.cpu()
    if kc is not None:
        res["k_cache"], res["v_cache"] = kc.cpu(), vc.cpu()
    return res
