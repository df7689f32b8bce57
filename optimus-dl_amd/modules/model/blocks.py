"""Transformer blocks whose ``nn.Linear`` members carry the names the reference
uses (optimus_dl/modules/model/blocks/attention.py:120-123 ``wq wk wv wo``;
blocks/mlp.py:47-49 ``w1 w2 c_proj``; :101-102,142-144 ``c_fc c_proj``).  Only
what the FP8 Linear path needs is here: plain PyTorch attention (SDPA), RoPE,
RMSNorm / LayerNorm.  These are the callers either side of the Linear, not a
re-implementation of the reference's model zoo."""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        xf = x.float()
        y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)
        return (y * self.weight.float()).to(x.dtype)


def rope_tables(head_dim: int, seq_len: int, theta: float, device) -> tuple[torch.Tensor, torch.Tensor]:
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float32) / head_dim))
    ang = torch.outer(torch.arange(seq_len, device=device, dtype=torch.float32), inv)
    return ang.cos(), ang.sin()


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    # x: [B, H, T, D]; rotate pairs (even, odd)
    xf = x.float()
    x1, x2 = xf[..., 0::2], xf[..., 1::2]
    c, s = cos[None, None], sin[None, None]
    out = torch.stack((x1 * c - x2 * s, x1 * s + x2 * c), dim=-1).flatten(-2)
    return out.to(x.dtype)


class CausalSelfAttention(nn.Module):
    def __init__(self, n_embd: int, n_head: int, n_kv_head: int | None = None, head_dim: int | None = None,
                 bias: bool = False, use_qk_norm: bool = False, rope: bool = True, rope_theta: float = 10000.0,
                 rmsnorm_eps: float = 1e-5):
        super().__init__()
        assert n_embd % n_head == 0
        self.n_head = n_head
        self.n_kv_head = n_kv_head or n_head
        self.head_dim = head_dim or n_embd // n_head
        self.rope, self.rope_theta = rope, rope_theta
        self.wq = nn.Linear(n_embd, n_head * self.head_dim, bias=bias)
        self.wk = nn.Linear(n_embd, self.n_kv_head * self.head_dim, bias=bias)
        self.wv = nn.Linear(n_embd, self.n_kv_head * self.head_dim, bias=bias)
        self.wo = nn.Linear(n_head * self.head_dim, n_embd, bias=bias)
        self.use_qk_norm = use_qk_norm
        if use_qk_norm:
            self.q_norm = RMSNorm(self.head_dim, eps=rmsnorm_eps)
            self.k_norm = RMSNorm(self.head_dim, eps=rmsnorm_eps)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        B, T_, _ = x.shape
        q = self.wq(x).view(B, T_, self.n_head, self.head_dim).transpose(1, 2)
        k = self.wk(x).view(B, T_, self.n_kv_head, self.head_dim).transpose(1, 2)
        v = self.wv(x).view(B, T_, self.n_kv_head, self.head_dim).transpose(1, 2)
        if self.use_qk_norm:
            q, k = self.q_norm(q), self.k_norm(k)
        if self.rope:
            cos, sin = rope_tables(self.head_dim, T_, self.rope_theta, x.device)
            q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
        if self.n_kv_head != self.n_head:
            rep = self.n_head // self.n_kv_head
            k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
        y = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        return self.wo(y.transpose(1, 2).reshape(B, T_, self.n_head * self.head_dim))


class SwiGLUMLP(nn.Module):
    def __init__(self, n_embd: int, intermediate_size: int | None = None, multiple_of: int = 256, bias: bool = False):
        super().__init__()
        if intermediate_size is None:
            hidden = int(2 * (4 * n_embd) / 3)
            hidden = multiple_of * ((hidden + multiple_of - 1) // multiple_of)
        else:
            hidden = intermediate_size
        self.w1 = nn.Linear(n_embd, hidden, bias=bias)
        self.w2 = nn.Linear(n_embd, hidden, bias=bias)
        self.c_proj = nn.Linear(hidden, n_embd, bias=bias)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.c_proj(F.silu(self.w1(x)) * self.w2(x))


class GELUMLP(nn.Module):
    def __init__(self, n_embd: int, intermediate_size: int | None = None, bias: bool = True):
        super().__init__()
        hidden = intermediate_size or 4 * n_embd
        self.c_fc = nn.Linear(n_embd, hidden, bias=bias)
        self.gelu = nn.GELU()
        self.c_proj = nn.Linear(hidden, n_embd, bias=bias)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.c_proj(self.gelu(self.c_fc(x)))


class LlamaBlock(nn.Module):
    """Pre-norm block: x + attn(ln_1(x)); x + mlp(ln_2(x))."""

    def __init__(self, n_embd: int, n_head: int, n_kv_head: int | None, intermediate_size: int | None,
                 use_qk_norm: bool = False, head_dim: int | None = None, eps: float = 1e-5, rope_theta: float = 10000.0):
        super().__init__()
        self.ln_1 = RMSNorm(n_embd, eps)
        self.attn = CausalSelfAttention(n_embd, n_head, n_kv_head, head_dim, bias=False, use_qk_norm=use_qk_norm,
                                        rope_theta=rope_theta, rmsnorm_eps=eps)
        self.ln_2 = RMSNorm(n_embd, eps)
        self.mlp = SwiGLUMLP(n_embd, intermediate_size)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        x = x + self.attn(self.ln_1(x))
        return x + self.mlp(self.ln_2(x))


class Qwen3Block(LlamaBlock):
    def __init__(self, n_embd: int, n_head: int, n_kv_head: int | None, intermediate_size: int | None,
                 head_dim: int | None = None, eps: float = 1e-6, rope_theta: float = 1e6):
        super().__init__(n_embd, n_head, n_kv_head, intermediate_size, use_qk_norm=True, head_dim=head_dim, eps=eps,
                         rope_theta=rope_theta)


class GPT2Block(nn.Module):
    def __init__(self, n_embd: int, n_head: int, bias: bool = True):
        super().__init__()
        self.ln_1 = nn.LayerNorm(n_embd, bias=bias)
        self.attn = CausalSelfAttention(n_embd, n_head, bias=bias, rope=False)
        self.ln_2 = nn.LayerNorm(n_embd, bias=bias)
        self.mlp = GELUMLP(n_embd, bias=bias)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        x = x + self.attn(self.ln_1(x))
        return x + self.mlp(self.ln_2(x))
