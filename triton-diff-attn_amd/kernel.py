"""Autograd wiring of the MI355X differential-attention kernels.

Host-side counterpart of the reference's `_diff_attention` (src/kernel.py:461-575): same class
name, same `apply` argument order, same 9-slot gradient tuple (a tenth, optional argument `causal`
-- masking is a feature the reference lists as missing, src/kernel.py:4 -- adds a tenth slot).  The work itself is done by the
hand-written HIP kernels in libdiffattn.so, reached through its C ABI; if the library is missing
the call raises -- there is no other path.
"""
import torch
from torch.autograd.function import once_differentiable

import _native

_SUPPORTED_D = (32, 64, 128)
_SEQ_MULTIPLE = 128
_FLAG_RMS_NORM = 1      # DIFFATTN_RMS_NORM
_FLAG_CAUSAL = 2        # DIFFATTN_CAUSAL
_FLAG_BF16 = 4          # DIFFATTN_BF16
_FLAG_LAMBDA_PER_HEAD = 8   # DIFFATTN_LAMBDA_PER_HEAD
_DTYPES = (torch.float16, torch.bfloat16)


def _check_inputs(Q1, Q2, K1, K2, V):
    names = ("q1", "q2", "k1", "k2", "v")
    for n, t in zip(names, (Q1, Q2, K1, K2, V)):
        if not torch.is_tensor(t):
            raise TypeError("%s must be a tensor" % n)
        if t.dtype not in _DTYPES:
            raise TypeError("%s must be float16 (like the reference, src/kernel.py:3-4) or bfloat16 (got %s)"
                            % (n, t.dtype))
        if t.dtype != Q1.dtype:
            raise TypeError("all inputs must have the same dtype (%s has %s, q1 has %s)" % (n, t.dtype, Q1.dtype))
        if t.dim() != 4:
            raise ValueError("%s must be [B,H,N,D] (got %d dims)" % (n, t.dim()))
    for n, t in zip(names, (Q1, Q2, K1, K2, V)):
        if not t.is_cuda:
            raise ValueError("%s must live on the GPU" % n)
        if t.device != Q1.device:
            raise ValueError("all inputs must be on the same device")
    B, H, N, D = Q1.shape
    for n, t in zip(names[1:4], (Q2, K1, K2)):
        if tuple(t.shape) != (B, H, N, D):
            raise ValueError("%s has shape %s, expected %s" % (n, tuple(t.shape), (B, H, N, D)))
    if tuple(V.shape) != (B, H, N, 2 * D):
        raise ValueError("v has shape %s, expected %s" % (tuple(V.shape), (B, H, N, 2 * D)))
    if D not in _SUPPORTED_D:
        raise ValueError("head dim %d unsupported; supported: %s" % (D, _SUPPORTED_D))
    if N < 1:
        raise ValueError("empty sequence")
    return B, H, N, D


def _pad_rows(t, n_pad):
    """[B,H,N,C] -> dense [B,H,n_pad,C] with zero rows appended (the tensor itself when nothing is missing)."""
    if t.size(2) == n_pad:
        return t.contiguous()
    return torch.nn.functional.pad(t, (0, 0, 0, n_pad - t.size(2)))


def _lambda_tensor(lambda_scale, device, dtype=torch.float16, num_heads=1):
    """The kernels read lambda from device memory (src/kernel.py:138), in the dtype of the tensors.  A
    python number is wrapped (a superset of the reference, whose float default cannot reach its kernel).
    A tensor holds one value, like the reference's, or one per head (`num_heads` values, more than one)."""
    if torch.is_tensor(lambda_scale):
        if lambda_scale.numel() not in (1, num_heads):
            raise ValueError("lambda_scale must have exactly one element, or one per head (%d)" % num_heads)
        return lambda_scale.detach().to(device=device, dtype=dtype).reshape(-1).contiguous()
    return torch.tensor([float(lambda_scale)], dtype=dtype, device=device)


def _ptr(t):
    return 0 if t is None else t.data_ptr()


class _diff_attention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, Q1, Q2, K1, K2, V, SM_SCALE, LAMBDA_SCALE, LAMBDA_INIT, rms_norm=False, causal=False):
        B, H, N, D = _check_inputs(Q1, Q2, K1, K2, V)
        lib = _native.lib()
        dev = Q1.device
        # The kernels work on multiples of 128 rows (like the reference's, src/kernel.py:527).  Other
        # lengths are padded with zero rows here; forward and backward ignore the padding keys, and a
        # padded query row has a zero upstream gradient, so it adds nothing to dK and dV.
        n_pad = -(-N // _SEQ_MULTIPLE) * _SEQ_MULTIPLE
        q1, q2, k1, k2, v = (_pad_rows(t, n_pad) for t in (Q1, Q2, K1, K2, V))
        lam = _lambda_tensor(LAMBDA_SCALE, dev, Q1.dtype, H)
        rms_norm = bool(rms_norm)
        flags = ((_FLAG_RMS_NORM if rms_norm else 0) | (_FLAG_CAUSAL if causal else 0)
                 | (_FLAG_BF16 if Q1.dtype == torch.bfloat16 else 0)
                 | (_FLAG_LAMBDA_PER_HEAD if lam.numel() > 1 else 0))

        y = torch.empty_like(v)
        # what only a backward reads (src/kernel.py:505 saves its counterparts unconditionally) is neither
        # allocated nor written when no input asks for a gradient, e.g. under torch.no_grad()
        differentiable = any(ctx.needs_input_grad)
        u2 = torch.empty_like(v) if differentiable else None
        stat = lambda: torch.empty((B, H, n_pad), device=dev, dtype=torch.float32)
        lse1, lse2 = (stat(), stat()) if differentiable else (None, None)
        rinv = stat() if (rms_norm and differentiable) else None

        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream().cuda_stream
            _native.check(lib.diffattn_forward_padded(
                q1.data_ptr(), q2.data_ptr(), k1.data_ptr(), k2.data_ptr(), v.data_ptr(),
                lam.data_ptr(), y.data_ptr(), _ptr(u2), _ptr(lse1), _ptr(lse2), _ptr(rinv),
                B, H, n_pad, N, D, float(SM_SCALE), float(LAMBDA_INIT), flags, stream))

        if differentiable:
            ctx.save_for_backward(q1, q2, k1, k2, v, y, u2, lse1, lse2, rinv, lam)
        ctx.SM_SCALE = float(SM_SCALE)
        ctx.LAMBDA_INIT = float(LAMBDA_INIT)
        ctx.FLAGS = flags
        ctx.N_VALID = N
        ctx.lambda_meta = (LAMBDA_SCALE.dtype, LAMBDA_SCALE.shape) if torch.is_tensor(LAMBDA_SCALE) else None
        return y if n_pad == N else y[:, :, :N].contiguous()

    @staticmethod
    @once_differentiable        # the gradients are plain kernel outputs: a second derivative raises
    def backward(ctx, dO):
        q1, q2, k1, k2, v, y, u2, lse1, lse2, rinv, lam = ctx.saved_tensors
        B, H, N, D = q1.shape
        lib = _native.lib()
        dev = q1.device
        if dO.dtype != q1.dtype:
            dO = dO.to(q1.dtype)
        dO = _pad_rows(dO, N)           # N is the padded length here
        n_valid = ctx.N_VALID

        # only the kernels whose outputs some input asked for are launched (stage bits of the C ABI:
        # 1 row preprocess, 2 d(lambda) reduction, 4 dK/dV, 8 dQ)
        need = ctx.needs_input_grad
        want_q, want_kv = need[0] or need[1], need[2] or need[3] or need[4]
        want_lam = ctx.lambda_meta is not None and need[6]
        stages = 1 | (2 if want_lam else 0) | (4 if want_kv else 0) | (8 if want_q else 0)
        dq1, dq2 = (torch.empty_like(q1), torch.empty_like(q2)) if want_q else (None, None)
        dk1, dk2, dv = (torch.empty_like(k1), torch.empty_like(k2), torch.empty_like(v)) if want_kv else (None,) * 3
        dlam = torch.empty(lam.numel(), device=dev, dtype=q1.dtype) if want_lam else None
        ws_bytes = lib.diffattn_backward_workspace_bytes(B, H, N, D, ctx.FLAGS)
        ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)

        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream().cuda_stream
            _native.check(lib.diffattn_backward_stages(
                q1.data_ptr(), q2.data_ptr(), k1.data_ptr(), k2.data_ptr(), v.data_ptr(), lam.data_ptr(),
                y.data_ptr(), u2.data_ptr(), lse1.data_ptr(), lse2.data_ptr(), _ptr(rinv), dO.data_ptr(),
                _ptr(dq1), _ptr(dq2), _ptr(dk1), _ptr(dk2), _ptr(dv), _ptr(dlam),
                ws.data_ptr(), ws_bytes, B, H, N, n_valid, D, ctx.SM_SCALE, ctx.LAMBDA_INIT, ctx.FLAGS, stages, stream))

        dlambda = None
        if want_lam:
            dtype, shape = ctx.lambda_meta
            dlambda = dlam.to(dtype).reshape(shape)
        if n_valid != N:
            dq1, dq2, dk1, dk2, dv = (None if t is None else t[:, :, :n_valid].contiguous()
                                      for t in (dq1, dq2, dk1, dk2, dv))
        # one slot per forward argument: nine, or ten when `causal` was passed
        return (dq1, dq2, dk1, dk2, dv, None, dlambda) + (None,) * (len(ctx.needs_input_grad) - 7)
