"""CPU-only checks: the C-ABI library loads and exports every symbol include/diffattn.h declares,
argument rejection works without a GPU, and the host wrappers validate their inputs."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "diffattn.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(diffattn_[a-z_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    assert declared_symbols() == sorted([
        "diffattn_abi_version", "diffattn_strerror", "diffattn_forward", "diffattn_forward_padded",
        "diffattn_backward_workspace_bytes", "diffattn_backward", "diffattn_backward_stages",
        "diffattn_backward_static", "diffattn_dropout_mask"])


def test_library_exports_every_declared_symbol():
    import _native
    lib = _native.lib()
    for name in declared_symbols():
        assert hasattr(lib, name), name
        assert name in _native.SYMBOLS, "binding table misses %s" % name
    assert lib.diffattn_abi_version() == 7 == _native.ABI_VERSION


def test_argument_rejection_needs_no_gpu():
    import _native
    lib = _native.lib()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf) & ~255
    p += 256
    args = lambda B, H, N, D: ([p] * 5 + [p, p, p, p, p, p] + [B, H, N, D, 0.125, 0.8, 1, None])
    assert lib.diffattn_forward(*([None] + args(1, 1, 128, 64)[1:])) == -1
    assert lib.diffattn_forward(*args(1, 1, 128, 48)) == -2
    assert lib.diffattn_forward(*args(0, 1, 128, 64)) == -2
    assert lib.diffattn_forward(*args(1 << 12, 1 << 10, 128, 64)) == -2      # more than 2^28 rows
    assert lib.diffattn_forward(*args(1, 1, 100, 64)) == -3
    bad = args(1, 1, 128, 64)
    bad[0] = p + 2
    assert lib.diffattn_forward(*bad) == -5
    bad = args(1, 1, 128, 64)
    bad[-2] = 1 << 12                             # unknown flag bit
    assert lib.diffattn_forward(*bad) == -6
    padded = lambda n_valid, layout=None, drop=None: [p] * 11 + [1, 1, 128, n_valid, 64, 0.125, 0.8, 1, layout, drop, None]
    assert lib.diffattn_forward_padded(*padded(0)) == -3
    assert lib.diffattn_forward_padded(*padded(129)) == -3
    assert lib.diffattn_backward_workspace_bytes(1, 1, 100, 64, 0) == 0
    assert lib.diffattn_backward_workspace_bytes(1, 1, 128, 48, 0) == 0
    assert lib.diffattn_backward_workspace_bytes(1, 1, 128, 64, 1 << 12) == 0     # unknown flag bit
    need = lib.diffattn_backward_workspace_bytes(2, 3, 256, 64, 1)
    rows = 2 * 3 * 256
    assert need >= rows * 128 * 2 + 4 * rows * 4
    bargs = [p] * 5 + [p, p, p, p, p, p, p] + [p] * 6 + [p, need - 1, 2, 3, 256, 64, 0.125, 0.8, 1, None]
    assert lib.diffattn_backward(*bargs) == -4
    bargs[19], bargs[-2] = need, 1 << 12
    assert lib.diffattn_backward(*bargs) == -6
    sargs = lambda n_valid, layout=None, drop=None: bargs[:23] + [n_valid, 64, 0.125, 0.8, 1, 15, layout, drop, None]
    assert lib.diffattn_backward_stages(*sargs(0)) == -3
    assert lib.diffattn_backward_stages(*sargs(257)) == -3
    # strides: multiples of 8 elements, rows at least as far apart as they are wide
    good = dict(qk_b=128 * 64, qk_h=64, qk_n=64, v_b=128 * 128, v_h=128, v_n=128,
                y_b=128 * 128, y_h=128, y_n=128, dy_b=128 * 128, dy_h=128, dy_n=128)
    for field, value in (("qk_n", 32), ("v_n", 132), ("y_h", -8), ("dy_b", 4)):
        lay = _native.Layout(**dict(good, **{field: value}))
        if not field.startswith("dy"):
            assert lib.diffattn_forward_padded(*padded(128, ctypes.byref(lay))) == -8, field
        assert lib.diffattn_backward_stages(*sargs(256, ctypes.byref(lay))) == -8, field
    # y, which is written, may not overlap itself
    padded2 = lambda layout: [p] * 11 + [2, 2, 128, 128, 64, 0.125, 0.8, 1, layout, None, None]
    for field in ("y_b", "y_h"):
        lay = _native.Layout(**dict(good, **{field: 0}))
        assert lib.diffattn_forward_padded(*padded2(ctypes.byref(lay))) == -8, field
    # Arguments that pass validation reach the launch, which fails with a positive HIP error code where there
    # is no GPU; the pointers here are host memory, so these calls are made only where nothing can run.
    if not torch.cuda.is_available():
        # the forward neither reads nor checks the strides of dy: a forward-only caller may leave them zero
        fwd_only = _native.Layout(**{k: (0 if k.startswith("dy") else v) for k, v in good.items()})
        assert lib.diffattn_forward_padded(*padded(128, ctypes.byref(fwd_only))) > 0
        assert lib.diffattn_forward_padded(*padded(128, ctypes.byref(_native.Layout(**dict(good, dy_b=4))))) > 0
        broadcast_v = _native.Layout(**dict(good, v_b=0))       # an input may be broadcast over the batch
        assert lib.diffattn_forward_padded(*padded2(ctypes.byref(broadcast_v))) > 0
        lam32 = padded(128)
        lam32[18] = 1 | 16                                      # DIFFATTN_RMS_NORM | DIFFATTN_LAMBDA_FP32
        assert lib.diffattn_forward_padded(*lam32) > 0
    for bad_p in (-0.1, 1.0, float("nan")):
        drop = _native.Dropout(bad_p, 1)
        assert lib.diffattn_forward_padded(*padded(128, None, ctypes.byref(drop))) == -9, bad_p
        assert lib.diffattn_backward_stages(*sargs(256, None, ctypes.byref(drop))) == -9, bad_p
    assert lib.diffattn_dropout_mask(p, 1, 1, 128, 2, ctypes.byref(_native.Dropout(0.5, 1)), None) == -2     # stream 0 or 1
    assert lib.diffattn_dropout_mask(p, 1, 1, 128, 0, None, None) == -1
    for code in (0, -1, -2, -3, -4, -5, -6, -7, -8, -9):
        assert len(lib.diffattn_strerror(code)) > 0


def test_host_validation_errors():
    from kernel import _check_inputs, _lambda_tensor

    class FakeCuda(torch.Tensor):
        pass

    t = lambda *s, dt=torch.float16: torch.zeros(*s, dtype=dt)
    with pytest.raises(TypeError):
        _check_inputs(t(1, 1, 128, 64, dt=torch.float32), *[t(1, 1, 128, 64)] * 3, t(1, 1, 128, 128))
    with pytest.raises(TypeError):   # fp16 and bf16 inputs cannot be mixed
        _check_inputs(t(1, 1, 128, 64, dt=torch.bfloat16), *[t(1, 1, 128, 64)] * 3, t(1, 1, 128, 128))
    with pytest.raises(ValueError):
        _check_inputs(t(1, 128, 64), *[t(1, 1, 128, 64)] * 3, t(1, 1, 128, 128))
    with pytest.raises(ValueError):  # CPU tensors are rejected: there is no CPU path
        _check_inputs(*[t(1, 1, 128, 64)] * 4, t(1, 1, 128, 128))
    with pytest.raises(ValueError):
        _lambda_tensor(torch.zeros(2), torch.device("cpu"))
    with pytest.raises(ValueError):   # neither one value nor one per head
        _lambda_tensor(torch.zeros(3), torch.device("cpu"), num_heads=4)
    per_head = _lambda_tensor(torch.tensor([[0.1], [0.2], [0.3]], dtype=torch.float16), torch.device("cpu"), num_heads=3)
    assert per_head.shape == (3,) and per_head.dtype == torch.float16
    # an fp32 lambda is read as fp32 (and gets an fp32 gradient); other types go through the tensors' dtype
    assert _lambda_tensor(torch.tensor([[0.1], [0.2], [0.3]]), torch.device("cpu"), num_heads=3).dtype == torch.float32
    assert _lambda_tensor(torch.tensor([0.5], dtype=torch.float64), torch.device("cpu"), torch.bfloat16).dtype == torch.bfloat16
    assert _lambda_tensor(0.5, torch.device("cpu"), torch.bfloat16).dtype == torch.bfloat16
    from kernel import _grad_like, _in_place, _is_dense, _strides_ok
    x = torch.arange(2 * 3 * 5 * 4, dtype=torch.float16).reshape(2, 3, 5, 4)
    wide = torch.zeros(2, 16, 3, 64, dtype=torch.float16)              # a [B,N,H,C] buffer seen as [B,H,N,C]
    view = wide.transpose(1, 2)
    assert _strides_ok(view) and _in_place(view) is view and not _is_dense(view) and _is_dense(wide)
    assert not _strides_ok(x.transpose(2, 3)) and _in_place(x.transpose(2, 3)).is_contiguous()    # last dim strided
    # a gradient buffer takes the layout of a permuted dense tensor; for a slice of a longer tensor it is a
    # compact buffer in the same dimension order: either way its own strides go to the kernels
    assert _grad_like(view).stride() == view.stride()
    sliced = _grad_like(wide[:, :8].transpose(1, 2)[:, :, :, :32])
    assert _strides_ok(sliced) and sliced.stride() == (8 * 3 * 32, 32, 3 * 32, 1)
    assert not _strides_ok(torch.zeros(2, 3, 5, 36, dtype=torch.float16)[..., :32])               # rows not 16-byte aligned
    lam = _lambda_tensor(0.25, torch.device("cpu"))
    assert lam.dtype == torch.float16 and lam.shape == (1,) and lam.item() == 0.25


def test_drop_in_signature_matches_reference():
    import inspect
    import layers
    from kernel import _diff_attention
    sig = inspect.signature(layers.MultiheadDiffAttnKernel)
    # the reference's eight parameters in the reference's order; the additions follow at the end
    assert list(sig.parameters) == ["q1", "q2", "k1", "k2", "v", "lambda_scale", "lambda_init", "rms_norm", "causal",
                                    "dropout_p", "dropout_seed"]
    assert sig.parameters["causal"].default is False and sig.parameters["dropout_p"].default == 0.0
    assert sig.parameters["lambda_scale"].default == -0.5
    assert sig.parameters["lambda_init"].default == 0.8
    assert sig.parameters["rms_norm"].default is False
    fsig = inspect.signature(_diff_attention.forward)
    assert list(fsig.parameters) == ["ctx", "Q1", "Q2", "K1", "K2", "V", "SM_SCALE", "LAMBDA_SCALE", "LAMBDA_INIT", "rms_norm",
                                     "causal", "dropout_p", "dropout_seed"]
    assert fsig.parameters["causal"].default is False
    assert issubclass(_diff_attention, torch.autograd.Function)
