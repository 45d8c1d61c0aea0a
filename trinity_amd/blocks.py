"""Host-side plans behind the generated modules' `forward`.

A plan fixes the parameters of one computation (taken from the IR and the
tensor-metadata constants), owns the scratch buffers the HIP library needs
beyond the caller's tensors, and calls the C ABI on torch's current stream.
Scratch is allocated on the first call only (the reference's drivers always
run warm-up calls before capturing a graph, convert_eval_rms.py:253-263), so
`forward` allocates nothing afterwards and is safe under graph capture.

Reference semantics (baseline/ref_rms.py:28-403) are the defaults: no softmax
scale, no causal mask, as many KV heads as query heads, RMSNorm without eps
or weight, KeyFormer temperature 1.5 with the noise passed as a tensor.  The
benchmark configurations override them through the constructor.
"""
import torch

from . import ext


def _f32_view(t, rows, cols, cache, key):
    """fp32 [rows, cols] buffer for the kernels; returns (buffer, needs_copy_back)."""
    if t.dtype == torch.float32:
        return t, False
    buf = cache.get(key)
    if buf is None or buf.shape != (rows, cols) or buf.device != t.device:
        buf = torch.empty(rows, cols, dtype=torch.float32, device=t.device)
        cache[key] = buf
    return buf, True


class AttentionPlan:
    """QKV projection + KV-cache append + attention (vanilla | keyformer | roco),
    optionally with PreNorm and/or QKNorm."""

    def __init__(self, variant="vanilla", M=None, N=None, D=None, H=None, P=0, prenorm=False, qknorm=False, tau=1.5,
                 scale=1.0, causal=False, n_kv_heads=None, eps=0.0, noise_seed=0, as_mean_var=False):
        if variant not in ("vanilla", "keyformer", "roco"):
            raise ValueError("unknown attention variant %r" % variant)
        self.variant, self.M, self.N, self.D, self.H, self.P = variant, M, N, D, H, P
        self.prenorm, self.qknorm, self.tau = prenorm, qknorm, tau
        self.scale, self.causal, self.n_kv_heads, self.eps = scale, causal, n_kv_heads, eps
        self.noise_seed, self.as_mean_var = noise_seed, as_mean_var
        self._cache = {}

    def _params(self, X, WK):
        S, N = X.shape
        if self.M is not None and S != self.M:
            raise ValueError("X has %d rows, the plan was built for M = %d" % (S, self.M))
        D = self.D
        H = self.H if self.H is not None else N // D
        Hkv = self.n_kv_heads if self.n_kv_heads is not None else WK.shape[1] // D
        return ext.attn_params(H, Hkv, D, S, kv_prefix=self.P, scale=self.scale, causal=self.causal,
                               rms_eps=self.eps, prenorm=self.prenorm, qknorm=self.qknorm, tau=self.tau,
                               noise_seed=self.noise_seed), S, N, H

    def _scratch(self, p, N, dev):
        need = ext.qkv_scratch_bytes(p, N)
        buf = self._cache.get("scratch")
        if buf is None or buf.numel() < need or buf.device != dev:
            buf = torch.empty(need, dtype=torch.uint8, device=dev)
            self._cache["scratch"] = buf
        return buf

    def run(self, X, WQ, WK, WV, O2, K_cache=None, V_cache=None, noise=None, C_out=None, C_out1=None, C_out2=None,
            norm_w=None, lse=None):
        p, S, N, H = self._params(X, WK)
        scratch = self._scratch(p, N, X.device)
        L = self.P + S
        if self.variant == "vanilla":
            ext.qkv_attention(X, norm_w, WQ, WK, WV, K_cache, V_cache, scratch, lse, O2, p)
        elif self.variant == "keyformer":
            if C_out is None:
                raise ValueError("keyformer needs the C_out buffer")
            score, back = _f32_view(C_out, H, L, self._cache, "score")
            ext.keyformer(X, norm_w, WQ, WK, WV, K_cache, V_cache, scratch, noise, O2, score, p)
            if back:
                C_out.copy_(score)
        else:
            if C_out1 is None or C_out2 is None:
                raise ValueError("roco needs the C_out1 and C_out2 buffers")
            s1, b1 = _f32_view(C_out1, H, L, self._cache, "s1")
            s2, b2 = _f32_view(C_out2, H, L, self._cache, "s2")
            ext.roco(X, norm_w, WQ, WK, WV, K_cache, V_cache, scratch, O2, s1, s2, p, as_mean_var=self.as_mean_var)
            if b1:
                C_out1.copy_(s1)
            if b2:
                C_out2.copy_(s2)


class FfnBlockPlan:
    """The reference-shaped FFN block: output projection + residual + RMSNorm +
    SwiGLU + down projection (+ residual + RMSNorm with `falcon_tail`)."""

    def __init__(self, falcon_tail=False):
        self.falcon_tail = falcon_tail
        self._cache = {}

    def _buf(self, key, given, shape, dtype, dev):
        if given is not None:
            return given
        b = self._cache.get(key)
        if b is None or tuple(b.shape) != tuple(shape) or b.device != dev:
            b = torch.empty(*shape, dtype=dtype, device=dev)
            self._cache[key] = b
        return b

    def run(self, O2, WO, X, WFF1a, WFF1b, WFF2, attn_O2=None, FF1=None, FF2=None, O_FF_norm=None):
        M, N = O2.shape
        F = WFF1a.shape[1]
        dev = O2.device
        attn = self._buf("attn", attn_O2, (M, N), torch.float16, dev)
        ff1 = self._buf("ff1", FF1, (M, F), torch.float16, dev)
        ff2 = self._buf("ff2", FF2, (M, N), torch.float16, dev)
        rows = self._buf("rows", None, (M,), torch.float32, dev)
        if self.falcon_tail and O_FF_norm is None:
            raise ValueError("the Falcon-shaped block needs the O_FF_norm buffer")
        ws_bytes = ext.ffn_workspace_bytes(M, N, F)  # non-zero for few rows (the reference's M = 16)
        ws = self._buf("ws", None, (ws_bytes,), torch.uint8, dev) if ws_bytes else None
        ext.ffn_block(O2, WO, X, WFF1a, WFF1b, WFF2, attn, rows, ff1, ff2, O_FF_norm if self.falcon_tail else None,
                      workspace=ws)


class RmsNormPlan:
    """Standalone RMSNorm (reference point: no eps, no weight)."""

    def __init__(self, eps=0.0):
        self.eps = eps

    def run(self, O_FF, O_FF_norm, weight=None):
        ext.rmsnorm(O_FF, weight, O_FF_norm, self.eps)


class FfnPlan:
    """The benchmark configuration's plain FFNs: SwiGLU (gate, up, down) or
    GELU (w1, w2).  The hidden activation is plan-owned scratch."""

    def __init__(self, activation="swiglu"):
        if activation not in ("swiglu", "gelu"):
            raise ValueError("activation must be swiglu or gelu")
        self.activation = activation
        self._hidden = None
        self._ws = None

    def run(self, X, W1, W2, out, W_up=None):
        T, F = X.shape[0], W1.shape[1]
        if self._hidden is None or tuple(self._hidden.shape) != (T, F) or self._hidden.device != X.device:
            self._hidden = torch.empty(T, F, dtype=torch.float16, device=X.device)
        ws_bytes = ext.ffn_workspace_bytes(T, X.shape[1], F)
        if ws_bytes and (self._ws is None or self._ws.numel() < ws_bytes or self._ws.device != X.device):
            self._ws = torch.empty(ws_bytes, dtype=torch.uint8, device=X.device)
        ws = self._ws if ws_bytes else None
        if self.activation == "swiglu":
            if W_up is None:
                raise ValueError("SwiGLU needs W_up")
            ext.ffn_swiglu(X, W1, W_up, W2, self._hidden, out, workspace=ws)
        else:
            ext.ffn_gelu(X, W1, W2, self._hidden, out, workspace=ws)
