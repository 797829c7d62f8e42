"""A differential-attention layer built on the fused kernel.

The reference stops at the functional operator (src/layers.py:10-26); its kernel header points to
the Differential Transformer paper (src/kernel.py:1) for the layer around it.  This module is that
layer: input projections, the re-parametrised lambda, the fused operator with its per-head RMSNorm
and (1 - lambda_init) scale, a learnable per-feature gain on the normalised heads, and the output
projection.  Attention is bidirectional unless `causal=True`; `attention_dropout` drops entries of
the two softmax maps while the module is in training mode.

  x [B, N, E]  ->  q, k [B, 2H, N, d],  v [B, H, N, 2d]      (E = 2 * H * d)
  lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + lambda_init       (one scalar per layer, or one per
                                                                head with per_head_lambda=True)
  heads  = gain * MultiheadDiffAttnKernel(q1, q2, k1, k2, v, lambda, lambda_init, rms_norm=True)
  y      = out_proj(concat heads)
"""
import math

import torch
from torch import nn

from layers import MultiheadDiffAttnKernel


def lambda_init_for_depth(depth: int) -> float:
    """The paper's schedule for the initial lambda of layer `depth` (0-based)."""
    return 0.8 - 0.6 * math.exp(-0.3 * depth)


class DiffAttn(nn.Module):
    def __init__(self, embed_dim: int, num_heads: int, depth: int = 0, attention=MultiheadDiffAttnKernel,
                 causal: bool = False, per_head_lambda: bool = False, attention_dropout: float = 0.0,
                 device=None, dtype=torch.float16):
        super().__init__()
        if embed_dim % (2 * num_heads) != 0:
            raise ValueError("embed_dim must be divisible by 2 * num_heads")
        self.embed_dim = embed_dim
        self.num_heads = num_heads
        self.head_dim = embed_dim // (2 * num_heads)      # d: q/k sub-head width; a value head is 2d wide
        self.lambda_init = lambda_init_for_depth(depth)
        self.attention = attention
        self.causal = causal
        self.attention_dropout = float(attention_dropout)     # on both softmax maps, in training mode only
        kw = dict(device=device, dtype=dtype)
        self.q_proj = nn.Linear(embed_dim, embed_dim, bias=False, **kw)
        self.k_proj = nn.Linear(embed_dim, embed_dim, bias=False, **kw)
        self.v_proj = nn.Linear(embed_dim, embed_dim, bias=False, **kw)
        self.out_proj = nn.Linear(embed_dim, embed_dim, bias=False, **kw)
        # the four lambda vectors live in fp32: their products go through exp()
        lam = dict(device=device, dtype=torch.float32)
        shape = (num_heads, self.head_dim) if per_head_lambda else (self.head_dim,)
        self.lambda_q1 = nn.Parameter(torch.empty(shape, **lam).normal_(0.0, 0.1))
        self.lambda_k1 = nn.Parameter(torch.empty(shape, **lam).normal_(0.0, 0.1))
        self.lambda_q2 = nn.Parameter(torch.empty(shape, **lam).normal_(0.0, 0.1))
        self.lambda_k2 = nn.Parameter(torch.empty(shape, **lam).normal_(0.0, 0.1))
        self.head_gain = nn.Parameter(torch.ones(2 * self.head_dim, **kw))

    def lambda_scale(self) -> torch.Tensor:
        lam = (torch.exp((self.lambda_q1 * self.lambda_k1).sum(-1))
               - torch.exp((self.lambda_q2 * self.lambda_k2).sum(-1)) + self.lambda_init)
        return lam.reshape(-1)      # [1], or [num_heads] with per_head_lambda

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        B, N, E = x.shape
        H, d = self.num_heads, self.head_dim
        # sub-heads 2h and 2h+1 of the q/k projections are the two softmax streams of head h
        q = self.q_proj(x).view(B, N, H, 2, d).permute(3, 0, 2, 1, 4)
        k = self.k_proj(x).view(B, N, H, 2, d).permute(3, 0, 2, 1, 4)
        v = self.v_proj(x).view(B, N, H, 2 * d).transpose(1, 2)
        # lambda stays in fp32: the operator then reads it unrounded and returns its gradient in fp32, which a
        # gradient scaler's loss scale cannot push out of range
        lam = self.lambda_scale()
        # views of the projection outputs: the operator reads them through their strides and returns the
        # heads in v's [B,N,H,2d] memory layout, so neither side of it copies
        heads = self.attention(q[0], q[1], k[0], k[1], v, lambda_scale=lam, lambda_init=self.lambda_init, rms_norm=True,
                               **({"causal": True} if self.causal else {}),
                               **({"dropout_p": self.attention_dropout} if self.training and self.attention_dropout else {}))
        heads = heads * self.head_gain
        return self.out_proj(heads.transpose(1, 2).reshape(B, N, E))
