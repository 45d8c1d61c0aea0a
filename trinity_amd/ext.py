"""ctypes binding of libtrinity_amd.so for torch tensors.

PyTorch is used for device memory and streams only: every function below
marshals `tensor.data_ptr()` / shape / strides into the C structs of
include/trinity_amd.h and calls the matching `tri_*` entry point on torch's
current HIP stream.  There is no CPU or eager fallback: a missing library or a
non-zero status raises.
"""
import ctypes
import math
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtrinity_amd.so")

TRI_F16, TRI_BF16, TRI_F32, TRI_U8, TRI_FP8_E4M3 = 0, 1, 2, 3, 4
_DTYPES = {torch.float16: TRI_F16, torch.bfloat16: TRI_BF16, torch.float32: TRI_F32, torch.uint8: TRI_U8,
           torch.float8_e4m3fn: TRI_FP8_E4M3}


class TriTensor(ctypes.Structure):
    _fields_ = [
        ("ptr", ctypes.c_void_p),
        ("shape", ctypes.c_int64 * 4),
        ("stride", ctypes.c_int64 * 4),
        ("ndim", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
    ]


class TriAttnParams(ctypes.Structure):
    _fields_ = [
        ("n_q_heads", ctypes.c_int32),
        ("n_kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("seq", ctypes.c_int32),
        ("kv_prefix", ctypes.c_int32),
        ("scale", ctypes.c_float),
        ("causal", ctypes.c_int32),
        ("rms_eps", ctypes.c_float),
        ("prenorm", ctypes.c_int32),
        ("qknorm", ctypes.c_int32),
        ("tau", ctypes.c_float),
        ("noise_seed", ctypes.c_uint64),
        ("kv_fp8", ctypes.c_int32),
        ("k_scale", ctypes.c_float),
        ("v_scale", ctypes.c_float),
    ]


class TrinityError(RuntimeError):
    def __init__(self, fn, status, text):
        super().__init__("%s failed: status %d (%s)" % (fn, status, text))
        self.status = status


_lib = None

# every exported symbol of include/trinity_amd.h
EXPORTS = [
    "tri_abi_version", "tri_status_string", "tri_prepare",
    "tri_rmsnorm", "tri_validate_rmsnorm",
    "tri_ffn_swiglu", "tri_validate_ffn_swiglu",
    "tri_gemm_workspace_bytes", "tri_ffn_workspace_bytes",
    "tri_gateup_swiglu", "tri_matmul",
    "tri_ffn_gelu", "tri_validate_ffn_gelu",
    "tri_ffn_block", "tri_validate_ffn_block",
    "tri_qkv_scratch_bytes",
    "tri_qkv_attention", "tri_validate_qkv_attention", "tri_qkv_attention_static",
    "tri_keyformer", "tri_validate_keyformer",
    "tri_roco", "tri_validate_roco",
    "tri_diag_issue_probe", "tri_diag_power_probe",
]


def lib():
    """Load libtrinity_amd.so (built in-tree by trinity_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libtrinity_amd.so is missing (%s); run `python -m trinity_amd.build` - there is no fallback path"
                % LIB_PATH
            )
        L = ctypes.CDLL(LIB_PATH)
        L.tri_status_string.restype = ctypes.c_char_p
        L.tri_status_string.argtypes = [ctypes.c_int]
        L.tri_qkv_scratch_bytes.restype = ctypes.c_int64
        L.tri_qkv_scratch_bytes.argtypes = [ctypes.c_void_p, ctypes.c_int64]
        _lib = L
    return _lib


def as_tri(t):
    """torch tensor (or None) -> TriTensor (or None).  No copies are made."""
    if t is None:
        return None
    if t.dtype not in _DTYPES:
        raise TypeError("unsupported dtype %s" % t.dtype)
    if t.dim() > 4:
        raise ValueError("at most 4 dimensions")
    s = TriTensor()
    s.ptr = t.data_ptr()
    for i in range(t.dim()):
        s.shape[i] = t.shape[i]
        s.stride[i] = t.stride(i)
    s.ndim = t.dim()
    s.dtype = _DTYPES[t.dtype]
    return s


def _ref(s):
    return ctypes.byref(s) if s is not None else None


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _check(fn, status):
    if status != 0:
        raise TrinityError(fn, status, lib().tri_status_string(status).decode())


def _call(name, args, validate_only):
    L = lib()
    keep = [as_tri(a) if isinstance(a, torch.Tensor) else a for a in args]
    cargs = [_ref(k) if isinstance(k, TriTensor) else k for k in keep]
    fn = getattr(L, name)
    fn.restype = ctypes.c_int
    st = fn(*cargs)
    if validate_only:
        return st
    _check(name, st)
    return st


def attn_params(n_q_heads, n_kv_heads, head_dim, seq, kv_prefix=0, scale=None, causal=True, rms_eps=0.0,
                prenorm=False, qknorm=False, tau=1.0, noise_seed=0, kv_fp8=False, k_scale=1.0, v_scale=1.0):
    p = TriAttnParams()
    p.n_q_heads, p.n_kv_heads, p.head_dim, p.seq, p.kv_prefix = n_q_heads, n_kv_heads, head_dim, seq, kv_prefix
    p.scale = (1.0 / math.sqrt(head_dim)) if scale is None else scale
    p.causal = int(bool(causal))
    p.rms_eps = rms_eps
    p.prenorm, p.qknorm = int(bool(prenorm)), int(bool(qknorm))
    p.tau = tau
    p.noise_seed = noise_seed
    p.kv_fp8, p.k_scale, p.v_scale = int(bool(kv_fp8)), k_scale, v_scale
    return p


def qkv_scratch_bytes(params, n_model=0):
    n = lib().tri_qkv_scratch_bytes(ctypes.byref(params), ctypes.c_int64(n_model))
    if n < 0:
        _check("tri_qkv_scratch_bytes", int(n))
    return int(n)


# --------------------------------------------------------------------------- entry points
def prepare():
    """Give every kernel that needs more than 64 KB of LDS that attribute on the current device (tri_prepare); a
    caller that captures its very first call into a graph does this once beforehand."""
    fn = lib().tri_prepare
    fn.restype = ctypes.c_int
    _check("tri_prepare", fn())


def rmsnorm(x, w, y, eps=0.0, validate_only=False):
    args = [x, w, y, ctypes.c_float(eps)]
    if validate_only:
        return _call("tri_validate_rmsnorm", args, True)
    return _call("tri_rmsnorm", args + [_stream(x)], False)


def gemm_workspace_bytes(m, k, ncols):
    """Bytes of split-K workspace for one [m, k] x [k, ncols] product (0: the few-row path is never taken)."""
    fn = lib().tri_gemm_workspace_bytes
    fn.restype = ctypes.c_int64
    return int(fn(ctypes.c_int64(m), ctypes.c_int64(k), ctypes.c_int64(ncols)))


def ffn_workspace_bytes(m, n, f):
    """Bytes of split-K workspace that serve every product of an FFN on x [m, n] with hidden width f."""
    fn = lib().tri_ffn_workspace_bytes
    fn.restype = ctypes.c_int64
    return int(fn(ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(f)))


def ffn_swiglu(x, w_gate, w_up, w_down, hidden, out, workspace=None, validate_only=False):
    args = [x, w_gate, w_up, w_down, hidden, out, workspace]
    if validate_only:
        return _call("tri_validate_ffn_swiglu", args, True)
    return _call("tri_ffn_swiglu", args + [_stream(x)], False)


def gateup_swiglu(x, w_gate, w_up, row_scale, hidden, workspace=None):
    return _call("tri_gateup_swiglu", [x, w_gate, w_up, row_scale, hidden, workspace, _stream(x)], False)


def matmul(x, w, residual, out, workspace=None):
    return _call("tri_matmul", [x, w, residual, out, workspace, _stream(x)], False)


def ffn_gelu(x, w1, w2, hidden, out, workspace=None, validate_only=False):
    args = [x, w1, w2, hidden, out, workspace]
    if validate_only:
        return _call("tri_validate_ffn_gelu", args, True)
    return _call("tri_ffn_gelu", args + [_stream(x)], False)


def ffn_block(o2, wo, x, wff1a, wff1b, wff2, attn_o2, row_scratch, ff1, ff2, o_ff_norm=None, workspace=None,
              validate_only=False):
    args = [o2, wo, x, wff1a, wff1b, wff2, attn_o2, row_scratch, ff1, ff2, o_ff_norm, workspace]
    if validate_only:
        return _call("tri_validate_ffn_block", args, True)
    return _call("tri_ffn_block", args + [_stream(x)], False)


def qkv_attention(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, lse, out, params, validate_only=False):
    args = [x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, lse, out, ctypes.byref(params)]
    if validate_only:
        return _call("tri_validate_qkv_attention", args, True)
    return _call("tri_qkv_attention", args + [_stream(x)], False)


STATIC_SCRATCH_BYTES = 64 * 1024 * 1024  # TRI_STATIC_SCRATCH_BYTES


def qkv_attention_static(x, norm_w, wq, wk, wv, k_cache, v_cache, lse, out, params, status_only=False):
    """tri_qkv_attention with the library's own per-GPU scratch array (nothing is allocated); with `status_only`
    the status is returned instead of raised."""
    stream = _stream(x) if x.is_cuda else None  # (host tensors: only to read the status of a call that is refused)
    args = [x, norm_w, wq, wk, wv, k_cache, v_cache, lse, out, ctypes.byref(params), stream]
    return _call("tri_qkv_attention_static", args, status_only)


def keyformer(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, noise, out, score, params, validate_only=False):
    args = [x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, noise, out, score, ctypes.byref(params)]
    if validate_only:
        return _call("tri_validate_keyformer", args, True)
    return _call("tri_keyformer", args + [_stream(x)], False)


def roco(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, out, sum_out, sumsq_out, params, as_mean_var=False,
         validate_only=False):
    args = [x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, out, sum_out, sumsq_out,
            ctypes.c_int32(int(bool(as_mean_var))), ctypes.byref(params)]
    if validate_only:
        return _call("tri_validate_roco", args, True)
    return _call("tri_roco", args + [_stream(x)], False)


def issue_probe(with_mfma, n_valu, n_trans, waves_per_simd, iters=4096, workgroups=256, device="cuda:0"):
    """tri_diag_issue_probe: (s_memtime ticks, nanoseconds) per group of one MFMA (or none), n_valu v_fma_f32 and
    n_trans v_exp_f32, from a workgroup's start to the end of its last wave, averaged over the workgroups (one per
    CU, 4 * waves_per_simd waves each)."""
    ticks = torch.zeros(workgroups * 16 + 16, dtype=torch.uint8, device=device)
    args = [ctypes.c_int32(int(bool(with_mfma))), ctypes.c_int32(n_valu), ctypes.c_int32(n_trans),
            ctypes.c_int32(waves_per_simd), ctypes.c_int32(iters), ctypes.c_int32(workgroups), ticks, _stream(ticks)]
    _call("tri_diag_issue_probe", args, False)
    torch.cuda.synchronize()
    t = ticks[: workgroups * 16].view(torch.int64).view(workgroups, 2).double().mean(0)
    return float(t[0]) / iters, float(t[1]) * 10.0 / iters


def power_probe(lds_reads_per_two_groups, dma_loads_per_eight_groups, n_valu, n_trans, random_operands,
                iters=1 << 20, workgroups=256, device="cuda:0"):
    """tri_diag_power_probe: (s_memtime ticks, nanoseconds, clock in GHz) of one SIMD per group of one MFMA with LDS
    reads, global -> LDS loads, v_fma_f32 and v_exp_f32 beside it - two waves per SIMD, so half a workgroup's loop time per group - on
    the second of two launches (the first brings the clock to where the load holds it)."""
    ticks = torch.zeros(workgroups * 16 + 16, dtype=torch.uint8, device=device)
    args = [ctypes.c_int32(lds_reads_per_two_groups), ctypes.c_int32(dma_loads_per_eight_groups),
            ctypes.c_int32(n_valu), ctypes.c_int32(n_trans),
            ctypes.c_int32(int(bool(random_operands))), ctypes.c_int32(iters), ctypes.c_int32(workgroups), ticks,
            _stream(ticks)]
    for _ in range(2):
        _call("tri_diag_power_probe", args, False)
        torch.cuda.synchronize()
    t = ticks[: workgroups * 16].view(torch.int64).view(workgroups, 2).double().mean(0)
    ns = float(t[1]) * 10.0
    return float(t[0]) / iters / 2, ns / iters / 2, float(t[0]) / ns
