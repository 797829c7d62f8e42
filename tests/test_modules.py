"""The differential-attention layer (modules.py): host-side structure on the CPU with the stock-PyTorch
operator plugged in, and on the GPU the same layer with the fused kernel against the stock operator."""
import copy
import math

import pytest
import torch

import baselines
import modules


def test_lambda_schedule_and_reparametrisation():
    assert modules.lambda_init_for_depth(0) == pytest.approx(0.2)
    assert modules.lambda_init_for_depth(10) == pytest.approx(0.8 - 0.6 * math.exp(-3.0))
    layer = modules.DiffAttn(64, 2, depth=3, attention=baselines.MultiheadDiffAttn, dtype=torch.float32)
    with torch.no_grad():
        layer.lambda_q1.fill_(0.5); layer.lambda_k1.fill_(0.25); layer.lambda_q2.fill_(-0.5); layer.lambda_k2.fill_(0.5)
    d = layer.head_dim
    want = math.exp(0.125 * d) - math.exp(-0.25 * d) + layer.lambda_init
    assert layer.lambda_scale().shape == (1,)
    assert layer.lambda_scale().item() == pytest.approx(want, rel=1e-5)


def test_layer_shapes_and_gradients_reach_every_parameter():
    torch.manual_seed(0)
    layer = modules.DiffAttn(64, 2, depth=1, attention=baselines.MultiheadDiffAttn, dtype=torch.float32)
    assert layer.head_dim == 16
    x = torch.randn(2, 24, 64, requires_grad=True)
    y = layer(x)
    assert y.shape == x.shape
    y.square().mean().backward()
    for name, p in layer.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all() and p.grad.abs().sum() > 0, name
    assert x.grad is not None
    with pytest.raises(ValueError):
        modules.DiffAttn(60, 4)


def test_layer_matches_a_direct_evaluation_of_its_formula():
    torch.manual_seed(1)
    layer = modules.DiffAttn(32, 2, depth=2, attention=baselines.MultiheadDiffAttn, dtype=torch.float32)
    x = torch.randn(1, 8, 32)
    B, N, E, H, d = 1, 8, 32, 2, 8
    q = layer.q_proj(x).view(B, N, 2 * H, d).transpose(1, 2)
    k = layer.k_proj(x).view(B, N, 2 * H, d).transpose(1, 2)
    v = layer.v_proj(x).view(B, N, H, 2 * d).transpose(1, 2)
    a = torch.softmax(q @ k.transpose(-1, -2) / math.sqrt(d), -1).view(B, H, 2, N, N)
    lam = layer.lambda_scale()
    heads = (a[:, :, 0] - lam * a[:, :, 1]) @ v
    heads = heads * torch.rsqrt(heads.square().mean(-1, keepdim=True) + 1e-5) * (1 - layer.lambda_init) * layer.head_gain
    want = layer.out_proj(heads.transpose(1, 2).reshape(B, N, E))
    assert torch.allclose(layer(x), want, atol=1e-5)


@pytest.mark.gpu
def test_layer_with_the_kernel_matches_the_stock_operator():
    torch.manual_seed(2)
    dev = torch.device("cuda:0")
    fused = modules.DiffAttn(512, 4, depth=2, device=dev)            # head_dim 64, fp16
    stock = copy.deepcopy(fused)
    stock.attention = baselines.MultiheadDiffAttn
    x = (0.5 * torch.randn(2, 256, 512, device=dev)).half()
    xs = [x.clone().requires_grad_(True) for _ in range(2)]
    ys = [m(xi) for m, xi in zip((fused, stock), xs)]
    assert (ys[0].float() - ys[1].float()).abs().max().item() <= 1e-2
    g = torch.randn_like(ys[0])
    for y in ys:
        y.backward(g)
    assert (xs[0].grad.float() - xs[1].grad.float()).abs().max().item() <= 2e-2 * xs[1].grad.float().abs().max().item() + 1e-3
    for (name, pf), (_, ps) in zip(fused.named_parameters(), stock.named_parameters()):
        scale = ps.grad.float().abs().max().item()
        assert (pf.grad.float() - ps.grad.float()).abs().max().item() <= 5e-2 * scale + 1e-3, name


@pytest.mark.gpu
def test_causal_layer_with_the_kernel_matches_the_stock_operator():
    torch.manual_seed(3)
    dev = torch.device("cuda:0")
    fused = modules.DiffAttn(256, 2, depth=1, causal=True, device=dev)
    stock = copy.deepcopy(fused)
    stock.attention = baselines.MultiheadDiffAttn
    x = (0.5 * torch.randn(1, 384, 256, device=dev)).half()
    y_f, y_s = fused(x), stock(x)
    assert (y_f.float() - y_s.float()).abs().max().item() <= 1e-2
    # a causal layer's output at position i does not change when later positions do
    x2 = x.clone(); x2[:, 200:] = 0
    assert (fused(x2)[:, :200].float() - y_f[:, :200].float()).abs().max().item() <= 2e-3


def test_per_head_lambda_layer():
    torch.manual_seed(4)
    one = modules.DiffAttn(64, 4, depth=2, attention=baselines.MultiheadDiffAttn, dtype=torch.float32)
    per = modules.DiffAttn(64, 4, depth=2, attention=baselines.MultiheadDiffAttn, per_head_lambda=True,
                           dtype=torch.float32)
    assert per.lambda_q1.shape == (4, 8) and per.lambda_scale().shape == (4,)
    # with every head given the single-lambda layer's vectors, the two layers are the same function
    state = one.state_dict()
    for name in ("lambda_q1", "lambda_k1", "lambda_q2", "lambda_k2"):
        state[name] = state[name].expand(4, -1).clone()
    per.load_state_dict(state)
    x = torch.randn(2, 12, 64)
    assert torch.allclose(per(x), one(x), atol=1e-6)
    # distinct per-head vectors give distinct lambdas, and each reaches the output
    with torch.no_grad():
        per.lambda_q1.copy_(torch.linspace(-0.5, 0.5, 32).reshape(4, 8))
    lam = per.lambda_scale()
    assert lam.unique().numel() == 4
    per(x).square().mean().backward()
    assert per.lambda_q1.grad.abs().sum(-1).min() > 0


@pytest.mark.gpu
def test_per_head_lambda_layer_with_the_kernel_matches_the_stock_operator():
    torch.manual_seed(5)
    dev = torch.device("cuda:0")
    fused = modules.DiffAttn(512, 4, depth=3, per_head_lambda=True, device=dev)
    with torch.no_grad():
        fused.lambda_q1.copy_(torch.linspace(-0.3, 0.3, 4 * 64).reshape(4, 64))
    stock = copy.deepcopy(fused)
    stock.attention = baselines.MultiheadDiffAttn
    x = (0.5 * torch.randn(2, 256, 512, device=dev)).half()
    xs = [x.clone().requires_grad_(True) for _ in range(2)]
    ys = [m(xi) for m, xi in zip((fused, stock), xs)]
    assert (ys[0].float() - ys[1].float()).abs().max().item() <= 1e-2
    g = torch.randn_like(ys[0])
    for y in ys:
        y.backward(g)
    for (name, pf), (_, ps) in zip(fused.named_parameters(), stock.named_parameters()):
        scale = ps.grad.float().abs().max().item()
        assert (pf.grad.float() - ps.grad.float()).abs().max().item() <= 5e-2 * scale + 1e-3, name


@pytest.mark.gpu
def test_attention_dropout_acts_in_training_mode_only():
    torch.manual_seed(6)
    dev = torch.device("cuda:0")
    layer = modules.DiffAttn(256, 2, attention_dropout=0.3, device=dev)
    x = (0.5 * torch.randn(2, 128, 256, device=dev)).half()
    layer.eval()
    a, b = layer(x), layer(x)
    assert torch.equal(a, b)
    layer.train()
    c, d = layer(x), layer(x)
    assert not torch.equal(c, d) and not torch.equal(c, a)      # fresh masks per call
    assert torch.isfinite(c).all()
    c.float().square().mean().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in layer.parameters())
