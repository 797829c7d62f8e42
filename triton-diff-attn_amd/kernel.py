"""Autograd wiring of the MI355X differential-attention kernels.

Host-side counterpart of the reference's `_diff_attention` (src/kernel.py:461-575): same class
name, same `apply` argument order, same 9-slot gradient tuple (the optional arguments `causal`,
`dropout_p` and `dropout_seed` -- masking and dropout are features the reference lists as missing,
src/kernel.py:4 -- add a slot each).  The work itself is done by the
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
_FLAG_LAMBDA_FP32 = 16      # DIFFATTN_LAMBDA_FP32
_FLAG_UNPADDED = 32         # DIFFATTN_UNPADDED
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


def _strides_ok(t):
    """Whether the kernels can read t in place: contiguous rows, every other stride a non-negative
    multiple of 8 elements (16-byte aligned rows), base pointer 16-byte aligned."""
    sb, sh, sn, sc = t.stride()
    return (sc == 1 and sn >= t.size(3) and sn % 8 == 0 and sb % 8 == 0 and sh % 8 == 0 and sb >= 0 and sh >= 0
            and sn <= (1 << 26) and t.data_ptr() % 16 == 0)


def _in_place(t):
    """t itself when the kernels can read it through its strides, else a dense copy."""
    return t if _strides_ok(t) else t.contiguous()


def _is_dense(t):
    B, H, N, C = t.shape
    return t.stride() == (H * N * C, N * C, C, 1)


def _grad_like(t):
    """An uninitialised gradient buffer in t's memory layout when t is a permuted dense buffer (autograd then
    takes it as it is instead of copying it into the leaf's layout), else dense."""
    return torch.empty_like(t)


def _current_stream(dev):
    """Raw handle of torch's current stream on dev (no Stream object is built)."""
    return torch._C._cuda_getCurrentRawStream(dev.index if dev.index is not None else torch._C._cuda_getDevice())


def _lambda_tensor(lambda_scale, device, dtype=torch.float16, num_heads=1):
    """The kernels read lambda from device memory (src/kernel.py:138).  A python number is wrapped, in the
    dtype of the tensors (a superset of the reference, whose float default cannot reach its kernel).
    A tensor holds one value, like the reference's, or one per head (`num_heads` values, more than one);
    an fp32 tensor is read as fp32 and gets an fp32 gradient, anything else goes through the tensors' dtype
    like the reference's `dtype=V.dtype` (src/kernel.py:573)."""
    if torch.is_tensor(lambda_scale):
        if lambda_scale.numel() not in (1, num_heads):
            raise ValueError("lambda_scale must have exactly one element, or one per head (%d)" % num_heads)
        if lambda_scale.dtype == torch.float32:
            dtype = torch.float32
        return lambda_scale.detach().to(device=device, dtype=dtype).reshape(-1).contiguous()
    return torch.tensor([float(lambda_scale)], dtype=dtype, device=device)


def _ptr(t):
    return 0 if t is None else t.data_ptr()


class _diff_attention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, Q1, Q2, K1, K2, V, SM_SCALE, LAMBDA_SCALE, LAMBDA_INIT, rms_norm=False, causal=False,
                dropout_p=0.0, dropout_seed=0):
        B, H, N, D = _check_inputs(Q1, Q2, K1, K2, V)
        dropout_p = float(dropout_p)
        if not 0.0 <= dropout_p <= 255 / 256:
            raise ValueError("dropout_p must lie in [0, 255/256] (got %r)" % dropout_p)
        # the same struct goes to the backward: the masks are a function of (seed, position) only
        dropout = _native.Dropout(dropout_p, int(dropout_seed) & 0xFFFFFFFFFFFFFFFF) if dropout_p > 0 else None
        lib = _native.lib()
        dev = Q1.device
        # The kernels work on blocks of 128 rows (like the reference's, src/kernel.py:527).  For other lengths
        # they run on the next multiple of 128, redirect reads past the last real row to that row and ignore
        # the padding keys: no tensor is padded or copied here; only what the library keeps for itself (u2,
        # the row statistics, the backward's workspace) is sized for the padded length.
        n_pad = -(-N // _SEQ_MULTIPLE) * _SEQ_MULTIPLE
        # Tensors are read through their strides (the reference passes Q1's and V's to its kernel,
        # src/kernel.py:487-494): a [B,N,H,d] projection output viewed as [B,H,N,d] is not copied.
        # The four q/k tensors share one set of strides, as in the reference.
        q1, q2, k1, k2, v = (_in_place(t) for t in (Q1, Q2, K1, K2, V))
        if not (q1.stride() == q2.stride() == k1.stride() == k2.stride()):
            q1, q2, k1, k2 = (t.contiguous() for t in (q1, q2, k1, k2))
        lam = _lambda_tensor(LAMBDA_SCALE, dev, Q1.dtype, H)
        rms_norm = bool(rms_norm)
        flags = ((_FLAG_RMS_NORM if rms_norm else 0) | (_FLAG_CAUSAL if causal else 0)
                 | (_FLAG_BF16 if Q1.dtype == torch.bfloat16 else 0)
                 | (_FLAG_LAMBDA_PER_HEAD if lam.numel() > 1 else 0)
                 | (_FLAG_LAMBDA_FP32 if lam.dtype == torch.float32 else 0)
                 | (_FLAG_UNPADDED if n_pad != N else 0))

        y = torch.empty_like(v)         # v's layout when v is a permuted dense buffer, else dense
        layout = None
        if not (_is_dense(q1) and _is_dense(v) and _is_dense(y)):
            layout = _native.Layout(*q1.stride()[:3], *v.stride()[:3], *y.stride()[:3], *y.stride()[:3])
        # what only a backward reads (src/kernel.py:505 saves its counterparts unconditionally) is neither
        # allocated nor written when no input asks for a gradient, e.g. under torch.no_grad()
        differentiable = any(ctx.needs_input_grad)
        u2 = lse1 = lse2 = rinv = None
        if differentiable:
            u2 = torch.empty((B, H, n_pad, 2 * D), device=dev, dtype=v.dtype)
            # the two logsumexps and the RMSNorm statistic share one allocation
            stats = torch.empty((3 if rms_norm else 2, B, H, n_pad), device=dev, dtype=torch.float32)
            lse1, lse2 = stats[0], stats[1]
            rinv = stats[2] if rms_norm else None

        if dev.index is not None and dev.index != torch._C._cuda_getDevice():
            with torch.cuda.device(dev):
                rc = lib.diffattn_forward_padded(
                    q1.data_ptr(), q2.data_ptr(), k1.data_ptr(), k2.data_ptr(), v.data_ptr(),
                    lam.data_ptr(), y.data_ptr(), _ptr(u2), _ptr(lse1), _ptr(lse2), _ptr(rinv),
                    B, H, n_pad, N, D, float(SM_SCALE), float(LAMBDA_INIT), flags, layout, dropout, _current_stream(dev))
        else:
            rc = lib.diffattn_forward_padded(
                q1.data_ptr(), q2.data_ptr(), k1.data_ptr(), k2.data_ptr(), v.data_ptr(),
                lam.data_ptr(), y.data_ptr(), _ptr(u2), _ptr(lse1), _ptr(lse2), _ptr(rinv),
                B, H, n_pad, N, D, float(SM_SCALE), float(LAMBDA_INIT), flags, layout, dropout, _current_stream(dev))
        _native.check(rc)

        if differentiable:
            ctx.save_for_backward(q1, q2, k1, k2, v, y, u2, lse1, lse2, rinv, lam)
        ctx.SM_SCALE = float(SM_SCALE)
        ctx.LAMBDA_INIT = float(LAMBDA_INIT)
        ctx.FLAGS = flags
        ctx.N_PAD = n_pad
        ctx.DROPOUT = dropout
        ctx.lambda_meta = (LAMBDA_SCALE.dtype, LAMBDA_SCALE.shape) if torch.is_tensor(LAMBDA_SCALE) else None
        return y

    @staticmethod
    @once_differentiable        # the gradients are plain kernel outputs: a second derivative raises
    def backward(ctx, dO):
        q1, q2, k1, k2, v, y, u2, lse1, lse2, rinv, lam = ctx.saved_tensors
        B, H, N, D = q1.shape
        n_pad = ctx.N_PAD
        lib = _native.lib()
        dev = q1.device
        if dO.dtype != q1.dtype:
            dO = dO.to(q1.dtype)
        dO = _in_place(dO)

        # only the kernels whose outputs some input asked for are launched (stage bits of the C ABI:
        # 1 row preprocess, 2 d(lambda) reduction, 4 dK/dV, 8 dQ)
        need = ctx.needs_input_grad
        want_q, want_kv = need[0] or need[1], need[2] or need[3] or need[4]
        want_lam = ctx.lambda_meta is not None and need[6]
        stages = 1 | (2 if want_lam else 0) | (4 if want_kv else 0) | (8 if want_q else 0)
        # Gradients are written in the memory layout of the tensors they belong to (autograd would otherwise
        # copy each one into its leaf's layout).  The four q/k gradients share one set of strides, like q1..k2.
        dq1 = dq2 = dk1 = dk2 = dv = None
        if want_q:
            dq1, dq2 = _grad_like(q1), _grad_like(q1)
        if want_kv:
            dk1, dk2, dv = _grad_like(q1), _grad_like(q1), _grad_like(v)
        gqk = dq1 if want_q else dk1        # (a view that is not a permuted dense buffer gets a dense gradient)
        layout = None
        if not (_is_dense(q1) and _is_dense(v) and _is_dense(y) and _is_dense(dO)):
            layout = _native.Layout(*q1.stride()[:3], *v.stride()[:3], *y.stride()[:3], *dO.stride()[:3],
                                    *(gqk.stride()[:3] if gqk is not None else (0, 0, 0)),
                                    *(dv.stride()[:3] if dv is not None else (0, 0, 0)))
        dlam = torch.empty(lam.numel(), device=dev, dtype=lam.dtype) if want_lam else None
        ws_bytes = lib.diffattn_backward_workspace_bytes(B, H, n_pad, D, ctx.FLAGS)
        ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)

        def launch():
            return lib.diffattn_backward_stages(
                q1.data_ptr(), q2.data_ptr(), k1.data_ptr(), k2.data_ptr(), v.data_ptr(), lam.data_ptr(),
                y.data_ptr(), u2.data_ptr(), lse1.data_ptr(), lse2.data_ptr(), _ptr(rinv), dO.data_ptr(),
                _ptr(dq1), _ptr(dq2), _ptr(dk1), _ptr(dk2), _ptr(dv), _ptr(dlam),
                ws.data_ptr(), ws_bytes, B, H, n_pad, N, D, ctx.SM_SCALE, ctx.LAMBDA_INIT, ctx.FLAGS, stages,
                layout, ctx.DROPOUT, _current_stream(dev))

        if dev.index is not None and dev.index != torch._C._cuda_getDevice():
            with torch.cuda.device(dev):
                rc = launch()
        else:
            rc = launch()
        _native.check(rc)

        dlambda = None
        if want_lam:
            dtype, shape = ctx.lambda_meta
            dlambda = dlam.to(dtype).reshape(shape)
        # one slot per forward argument: nine, or more when causal / dropout arguments were passed
        return (dq1, dq2, dk1, dk2, dv, None, dlambda) + (None,) * (len(ctx.needs_input_grad) - 7)
