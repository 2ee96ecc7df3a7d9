"""Llama-style decoder layer whose seven linears run on the INT8 path (forward and backward):
the training step either side of the hot path, as BASELINE config 5 describes it (hidden 4096,
32 heads, MLP 14336, bf16 elsewhere).  RMSNorm, rotary embedding, causal attention (torch
SDPA) and SwiGLU stay in bf16; ``int8=False`` builds the bf16 twin used for loss/grad parity.
"""
import math

import torch
import torch.nn.functional as F

from .linear import Int8Linear

__all__ = ["DecoderLayer", "rope_tables"]


def rope_tables(seq_len, head_dim, device, base=10000.0):
    inv = 1.0 / (base ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float32) / head_dim))
    ang = torch.outer(torch.arange(seq_len, device=device, dtype=torch.float32), inv)
    return ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)


def _rope(x, cos, sin):
    # x: [B, H, S, D]; rotate pairs (even, odd halves convention)
    d = x.shape[-1] // 2
    x1, x2 = x[..., :d], x[..., d:]
    c, s = cos[None, None], sin[None, None]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


class RMSNorm(torch.nn.Module):
    def __init__(self, dim, eps=1e-5, device=None):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.ones(dim, device=device, dtype=torch.bfloat16))
        self.eps = eps

    def forward(self, x):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)).to(x.dtype) * self.weight


class DecoderLayer(torch.nn.Module):
    def __init__(self, hidden=4096, heads=32, mlp=14336, int8=True, scheme="block_channel", device=None):
        super().__init__()
        assert hidden % heads == 0
        self.hidden, self.heads, self.head_dim = hidden, heads, hidden // heads

        def lin(i, o):
            if int8:
                return Int8Linear(i, o, bias=False, scheme=scheme, device=device)
            m = torch.nn.Linear(i, o, bias=False, device=device, dtype=torch.bfloat16)
            torch.nn.init.normal_(m.weight, std=0.02)
            return m

        self.q_proj, self.k_proj, self.v_proj, self.o_proj = lin(hidden, hidden), lin(hidden, hidden), lin(hidden, hidden), lin(hidden, hidden)
        self.gate_proj, self.up_proj, self.down_proj = lin(hidden, mlp), lin(hidden, mlp), lin(mlp, hidden)
        self.input_norm, self.post_norm = RMSNorm(hidden, device=device), RMSNorm(hidden, device=device)

    def copy_weights_from(self, other):
        """Share initial values with another layer (int8 layer <-> bf16 twin)."""
        with torch.no_grad():
            for (_, p), (_, q) in zip(sorted(self.named_parameters()), sorted(other.named_parameters())):
                p.copy_(q)

    def forward(self, x):
        B, S, H = x.shape
        cos, sin = rope_tables(S, self.head_dim, x.device)
        h = self.input_norm(x)
        q = self.q_proj(h).view(B, S, self.heads, self.head_dim).transpose(1, 2)
        k = self.k_proj(h).view(B, S, self.heads, self.head_dim).transpose(1, 2)
        v = self.v_proj(h).view(B, S, self.heads, self.head_dim).transpose(1, 2)
        q, k = _rope(q, cos, sin), _rope(k, cos, sin)
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=1.0 / math.sqrt(self.head_dim))
        x = x + self.o_proj(a.transpose(1, 2).reshape(B, S, H))
        h = self.post_norm(x)
        return x + self.down_proj(F.silu(self.gate_proj(h)) * self.up_proj(h))
