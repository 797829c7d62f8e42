"""Drop-in for the hot path of the reference's `layers` module (src/layers.py:10-26)."""
import math

import torch

from kernel import _diff_attention
# stock-PyTorch comparison lines under the names the reference's benchmark imports from this
# module (src/benchmark.py:11-17); none of them is used by MultiheadDiffAttnKernel
from baselines import MultiheadAttn, MultiheadDiffAttn, MultiheadFlashAttn, MultiheadFlashDiffAttn  # noqa: F401


def MultiheadDiffAttnKernel(
    q1: torch.Tensor,
    q2: torch.Tensor,
    k1: torch.Tensor,
    k2: torch.Tensor,
    v: torch.Tensor,
    lambda_scale=-0.5,
    lambda_init: float = 0.8,
    rms_norm: bool = False,
    causal: bool = False,
    dropout_p: float = 0.0,
    dropout_seed=None,
):
    """(softmax(q1 k1^T / sqrt(d)) - lambda_scale * softmax(q2 k2^T / sqrt(d))) v, optionally followed
    by a per-row RMSNorm over the 2d output features and a (1 - lambda_init) scale.

    q1, q2, k1, k2: [B, H, N, d] fp16 on the GPU; v: [B, H, N, 2d]; lambda_scale: 1-element tensor
    (a python float is accepted too; a tensor of H elements gives every head its own lambda, which
    the reference does not have).  Returns [B, H, N, 2d] fp16 with autograd support for the
    five tensors and lambda_scale.  `causal` (not in the reference, which lists masking as missing,
    src/kernel.py:4) lets query i attend to keys 0..i only.  `dropout_p` (likewise missing in the
    reference) drops every entry of each of the two softmax maps independently with that
    probability, in steps of 1/256, and scales the kept ones by 1/(1-p); the masks are a function of
    `dropout_seed` (drawn from torch's default CPU generator when None) and the position.  The seed
    travels as a launch argument: a HIP graph captured around the call replays the same masks, so a call
    under capture has to name its seed.
    """
    head_dim = q1.size(-1)
    sm_scale = 1 / math.sqrt(head_dim)
    if dropout_p:
        if dropout_seed is None:
            # The seed is a host value handed to the kernels with the launch: under stream capture it would be
            # frozen into the graph and every replay would drop the same entries.
            if q1.is_cuda and torch.cuda.is_current_stream_capturing():
                raise RuntimeError("dropout under stream capture needs an explicit dropout_seed (the same masks are "
                                   "then applied on every replay of the graph)")
            dropout_seed = int(torch.randint(0, 2 ** 62, (1,)).item())
        return _diff_attention.apply(q1, q2, k1, k2, v, sm_scale, lambda_scale, lambda_init, rms_norm, bool(causal),
                                     float(dropout_p), int(dropout_seed))
    if causal:
        return _diff_attention.apply(q1, q2, k1, k2, v, sm_scale, lambda_scale, lambda_init, rms_norm, True)
    return _diff_attention.apply(q1, q2, k1, k2, v, sm_scale, lambda_scale, lambda_init, rms_norm)
