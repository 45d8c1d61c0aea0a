"""PyTorch-eager comparison modules, same names and constructor arguments as
the reference's baseline/ref_rms.py (:28-403) and baseline/ffn_ref.py (:12-52).

They run wherever their tensors live (torch ops on the GPU in the drivers) and
exist only so that the drivers can print the same "kernel vs eager" check the
reference prints; the HIP path never calls them.  Unlike the reference's
classes they return the KeyFormer / RoCo score tensors they compute.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F


class _EagerAttention(nn.Module):
    prenorm = False
    qknorm = False
    variant = "vanilla"

    def __init__(self, M, N, D, P, cache_K, cache_V, W_q=None, W_k=None, W_v=None, noise=None, tau=1.5):
        super().__init__()
        self.M, self.N, self.D, self.P, self.H = M, N, D, P, N // D
        self.W_q, self.W_k, self.W_v = W_q, W_k, W_v
        self.cache_K, self.cache_V = cache_K, cache_V
        self.noise, self.tau = noise, tau
        self.extras = {}

    def forward(self, X):
        if self.prenorm:
            X = X * torch.rsqrt(X.pow(2).mean(-1, keepdim=True))
        heads = lambda t: t.view(self.M, -1, self.D).transpose(0, 1)
        q, k, v = heads(X @ self.W_q), heads(X @ self.W_k), heads(X @ self.W_v)
        if self.qknorm:
            q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True))
            k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True))
        keys = torch.cat([self.cache_K[:, : self.P], k], dim=1)
        vals = torch.cat([self.cache_V[:, : self.P], v], dim=1)
        scores = q @ keys.transpose(1, 2)
        weights = F.softmax(scores, dim=-1)
        if self.variant == "keyformer":
            self.extras["C_out"] = F.softmax((scores + self.noise) / self.tau, dim=-1).sum(dim=1)
        elif self.variant == "roco":
            self.extras["C_out1"] = weights.sum(dim=1)
            self.extras["C_out2"] = weights.pow(2).sum(dim=1)
        return (weights @ vals).transpose(0, 1).contiguous().view(self.M, -1)


class Vanilla(_EagerAttention):
    pass


class PreNorm(_EagerAttention):
    prenorm = True


class QKNorm(_EagerAttention):
    qknorm = True


class NormQKNorm(_EagerAttention):
    prenorm = qknorm = True


class KeyFormer(_EagerAttention):
    variant = "keyformer"

    def __init__(self, M, N, D, P, noise, cache_K, cache_V, W_q=None, W_k=None, W_v=None, tau=1.5):
        super().__init__(M, N, D, P, cache_K, cache_V, W_q, W_k, W_v, noise=noise, tau=tau)


class NormKeyFormer(KeyFormer):
    prenorm = True


class RoCo(_EagerAttention):
    variant = "roco"


class NormRoCo(RoCo):
    prenorm = True


class SimpleFFN(nn.Module):
    def __init__(self, M, N, P, WO=None, WFF1a=None, WFF1b=None, WFF2=None, falcon_tail=False):
        super().__init__()
        self.M, self.N, self.P = M, N, P
        self.WO, self.WFF1a, self.WFF1b, self.WFF2 = WO, WFF1a, WFF1b, WFF2
        self.falcon_tail = falcon_tail

    def forward(self, O2, X):
        attn = O2 @ self.WO + X
        norm = attn / torch.sqrt(attn.pow(2).sum(dim=1, keepdim=True) / self.N)
        ff1 = (norm @ self.WFF1a) * F.silu(norm @ self.WFF1b)
        ff2 = ff1 @ self.WFF2
        if not self.falcon_tail:
            return ff2
        o_ff = ff2 + norm
        return o_ff / torch.sqrt(o_ff.pow(2).sum(dim=1, keepdim=True) / self.N)
