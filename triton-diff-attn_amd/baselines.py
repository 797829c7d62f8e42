"""Comparison lines for the benchmark sweep: the same operators written with stock PyTorch ops.

These are NOT the product path and nothing in `layers.MultiheadDiffAttnKernel` or `kernel.py` calls
them.  They exist so that the sweep in `benchmark.py` can show the fused kernel next to what a user
would otherwise run on this GPU, under the names the reference's benchmark uses
(src/benchmark.py:11-17, 105-116):

  MultiheadAttn            plain softmax attention, score matrix materialised   (src/layers.py:29-46)
  MultiheadDiffAttn        differential attention, score matrices materialised  (src/layers.py:49-80)
  MultiheadFlashAttn       plain attention through a fused library kernel       (src/layers.py:83-101)
  MultiheadFlashDiffAttn   differential attention as four fused-attention calls (src/layers.py:104-148)

The reference's two "Flash" lines call the flash-attn CUDA wheel, which does not exist for this GPU;
here they call `torch.nn.functional.scaled_dot_product_attention`, the fused attention that ships
with PyTorch-ROCm.  The reference's RMSNorm is apex `FusedRMSNorm(elementwise_affine=False)`;
here it is `torch.nn.functional.rms_norm` with the same eps (1e-5).
"""
import math

import torch
import torch.nn.functional as F

RMS_EPS = 1e-5


def _rms(x: torch.Tensor) -> torch.Tensor:
    return F.rms_norm(x, (x.size(-1),), eps=RMS_EPS)


def _per_head(lambda_scale, dtype=None):
    """A lambda tensor with one value per head broadcasts over [B, H, N, *]; one value or a number stays.
    A tensor is brought to the dtype of the probabilities it multiplies (an fp32 lambda would otherwise
    promote them and then meet v in another dtype)."""
    if torch.is_tensor(lambda_scale):
        if dtype is not None:
            lambda_scale = lambda_scale.to(dtype)
        if lambda_scale.numel() > 1:
            return lambda_scale.reshape(1, -1, 1, 1)
    return lambda_scale


def _probabilities(q: torch.Tensor, k: torch.Tensor, causal: bool = False) -> torch.Tensor:
    """softmax(q k^T / sqrt(d)) with the softmax in fp32 and the result back in the input dtype."""
    scores = (q @ k.transpose(-1, -2)) * (1.0 / math.sqrt(q.size(-1)))
    if causal:
        n = scores.size(-1)
        scores = scores.masked_fill(torch.ones(n, n, dtype=torch.bool, device=scores.device).triu(1), float("-inf"))
    return torch.softmax(scores.float(), dim=-1).to(q.dtype)


def MultiheadAttn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, rms_norm: bool = False):
    out = _probabilities(q, k) @ v
    return _rms(out) if rms_norm else out


def MultiheadDiffAttn(q1, q2, k1, k2, v, lambda_scale=-0.5, lambda_init: float = 0.8, rms_norm: bool = False,
                      causal: bool = False):
    weights = _probabilities(q1, k1, causal) - _per_head(lambda_scale, q1.dtype) * _probabilities(q2, k2, causal)
    out = weights @ v
    if rms_norm:
        out = (1 - lambda_init) * _rms(out)
    return out


def MultiheadFlashAttn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, rms_norm: bool = False):
    out = F.scaled_dot_product_attention(q, k, v)
    return _rms(out) if rms_norm else out


def MultiheadFlashDiffAttn(q1, q2, k1, k2, v, lambda_scale=-0.5, lambda_init: float = 0.8, rms_norm: bool = False,
                           causal: bool = False):
    # fused attention kernels want equal head dims for q, k and v: each stream runs once per half of v
    halves = v.split(q1.size(-1), dim=-1)
    stream1 = torch.cat([F.scaled_dot_product_attention(q1, k1, h, is_causal=causal) for h in halves], dim=-1)
    stream2 = torch.cat([F.scaled_dot_product_attention(q2, k2, h, is_causal=causal) for h in halves], dim=-1)
    out = stream1 - _per_head(lambda_scale, q1.dtype) * stream2
    if rms_norm:
        out = (1 - lambda_init) * _rms(out)
    return out
