"""CPU oracle for the fused-block path.  TEST INFRASTRUCTURE ONLY.

This package restates, on the CPU, the arithmetic of the reference's eager
PyTorch baselines (baseline/ref_rms.py:28-403, baseline/ffn_ref.py:12-52 and
:114-121) with the parameter superset the HIP kernels accept (softmax scale,
causal mask, cached-key prefix, grouped KV heads, RMSNorm eps/weight, Gumbel
noise).  Only tests, the smoke check and the benchmark's CPU-baseline leg may
import it; the shipped package never does, and never falls back to it.

How each function is pinned (the reference holds no stored vectors for this
path, so the pins are mathematical):

* rmsnorm           - torch.nn.functional.rms_norm, constant-row closed form,
                      scale invariance (tests/test_oracle.py)
* ffn_swiglu/gelu   - fp64 matmul + F.silu / F.gelu(approximate="none")
* ffn_block         - composition of the pinned pieces (residual, rmsnorm, swiglu)
* qkv_attention O2  - F.scaled_dot_product_attention with repeat_interleave for
                      grouped heads, a brute-force triple loop on tiny inputs,
                      row-sum-to-one and key-permutation invariance
* attention_stage   - equality with qkv_attention's O2 on that function's own q, k, v
* RoCo s1/s2        - uniform-attention closed forms (harmonic tail under the
                      causal mask), sum_k s1 = S, s2 <= s1
* KeyFormer score   - brute-force loops with a noise tensor at tau = 1.5 over a cached
                      prefix (causal and not), the zero-logit closed form
                      softmax(g / tau).sum(queries) for tensor and seeded noise,
                      tau / noise sensitivity, sum_k score = S
* philox4x32        - Random123's published known-answer vectors for seven rounds (what the kernels use) and ten
* gumbel_noise      - float stage: parity unpinned by any external vector (it is
                      this build's own definition: sixteen bits per key,
                      u = (bits + 0.5) * 2^-16, g = -log(-log(u))); the
                      distribution's mean / variance, the bit-to-key layout and
                      the independence of neighbouring keys are checked

The reference discards its KeyFormer/RoCo score tensors
(baseline/ref_rms.py:164-166, :351-352), so for those outputs this oracle *is*
the definition, following the discarded lines.
"""
from .blocks import (  # noqa: F401
    rmsnorm,
    ffn_swiglu,
    ffn_gelu,
    ffn_block,
    qkv_attention,
    attention_stage,
)
from .philox import philox4x32, philox4x32_10, gumbel_noise, uniform_from_bits  # noqa: F401
