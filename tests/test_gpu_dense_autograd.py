"""The dense FP8 layers as autograd functions (FP8Linear, FP8KeepXLinear, FP8MlpFunction,
FusedNormFP8MLPFunction) and the two operators they add to the path (RMSNorm with its gradient,
swiglu_grad).  Floating-point kernels: checked against float64 / torch fp32 references within
stated tolerances, and against the already-verified building blocks for exact consistency."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

# e4m3 keeps 3 mantissa bits: up to 2^-4 = 6.25% relative error per operand element, ~3.6% rms.  A GEMM
# with both operands quantised lands at 4-5% relative Frobenius error against exact math; every
# further quantised GEMM stage in a chain adds about as much again in quadrature.
FP8_REL = 0.06      # one FP8 GEMM stage
FP8_REL2 = 0.10     # two chained stages (MLP forward)
FP8_REL3 = 0.15     # three (MLP input / weight gradients)
BF16_REL = 8e-3     # one bf16 rounding on top of fp32 math


def rel(a, b):
    a, b = a.detach().double(), b.detach().double()
    return float(((a - b).norm() / (b.norm() + 1e-30)).detach())


@pytest.fixture(scope="module")
def U():
    from paddleformers_amd import _lib
    from paddleformers_amd import fp8_utils

    _lib.lib()
    return fp8_utils


def bf(shape, std=1.0, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, device="cuda", generator=g) * std).to(torch.bfloat16)


@pytest.mark.parametrize("M,H", [(5, 128), (300, 1408), (512, 7168)])
def test_rms_norm_forward_and_backward(U, M, H):
    from paddleformers_amd import functional as F8

    x, w, dy = bf((M, H), seed=1), (bf((H,), 0.1, seed=2).float() + 1).to(torch.bfloat16), bf((M, H), seed=3)
    eps = 1e-6
    y, invar = F8.fused_rms_norm_ext(x, w, eps)
    xd = x.double().requires_grad_(True)
    wd = w.double().requires_grad_(True)
    iv = torch.rsqrt((xd * xd).mean(dim=-1, keepdim=True) + eps)
    yd = xd * iv * wd
    assert rel(invar, iv.squeeze(-1)) < 1e-6
    assert rel(y, yd) < BF16_REL and float(((y.double() - yd).abs().max() / yd.abs().max()).detach()) < 2.0**-7
    yd.backward(dy.double())
    dx, dw = F8.fused_rms_norm_ext_grad(x, w, invar, dy, eps)
    assert dw.dtype == torch.float32 and dw.shape == (H,)
    assert rel(dx, xd.grad) < BF16_REL
    assert rel(dw, wd.grad) < 1e-5
    # 3-D input keeps its shape
    y3, iv3 = F8.fused_rms_norm_ext(x.reshape(1, M, H), w, eps)
    assert y3.shape == (1, M, H) and iv3.shape == (1, M) and torch.equal(y3.reshape(M, H), y)


def test_swiglu_grad_matches_autograd(U):
    from paddleformers_amd import functional as F8

    M, I = 200, 256
    o1, do2 = bf((M, 2 * I), seed=4), bf((M, I), seed=5)
    o1d = o1.double().requires_grad_(True)
    (torch.nn.functional.silu(o1d[:, :I]) * o1d[:, I:]).backward(do2.double())
    do1, none = F8.swiglu_grad(o1, None, do2)
    assert none is None and do1.shape == o1.shape and rel(do1, o1d.grad) < BF16_REL
    with pytest.raises(ValueError):
        F8.swiglu_grad(o1[:, :I], o1[:, I:], do2)


@pytest.mark.parametrize("keep_x", [False, True])
def test_fp8_linear_forward_backward(U, keep_x):
    In, Out, B, S = 512, 384, 2, 256
    layer = (U.FP8KeepXLinear if keep_x else U.FP8Linear)(In, Out, device="cuda")
    with torch.no_grad():
        layer.weight.copy_(bf((In, Out), 0.05, seed=6))
    x = bf((B, S, In), seed=7).requires_grad_(True)
    out = layer(x)
    assert out.shape == (B, S, Out) and out.dtype == torch.bfloat16
    # forward is exactly the verified building block
    ref_fwd = U.FP8LinearFunctionBase.compute_fp8_linear(x.detach().reshape(-1, In), layer.weight, weight_transpose=True,
                                                         return_transpose_only=True)
    assert torch.equal(out.reshape(-1, Out), ref_fwd)
    dout = bf((B, S, Out), seed=8)
    out.backward(dout)
    xr = x.detach().double().requires_grad_(True)
    wr = layer.weight.detach().double().requires_grad_(True)
    (xr @ wr).backward(dout.double())
    assert rel(out, (xr @ wr).detach()) < FP8_REL
    assert x.grad.shape == x.shape and rel(x.grad, xr.grad) < FP8_REL
    assert layer.weight.grad is None                      # the weight gradient goes to the fp32 accumulator
    assert layer.weight.main_grad.dtype == torch.float32 and rel(layer.weight.main_grad, wr.grad) < FP8_REL
    # a second backward accumulates
    first = layer.weight.main_grad.clone()
    layer(x).backward(dout)
    assert rel(layer.weight.main_grad, 2 * first) < 1e-6


@pytest.mark.parametrize("recompute", [False, True])
def test_fp8_mlp_function(U, recompute):
    H, I, M = 512, 256, 512
    mlp = U.FP8Mlp(H, I, device="cuda", recompute_fwd_gate_up=recompute)
    with torch.no_grad():
        mlp.w1.copy_(bf((H, 2 * I), 0.05, seed=9))
        mlp.w2.copy_(bf((I, H), 0.05, seed=10))
    x = bf((M, H), seed=11).requires_grad_(True)
    out = mlp(x)
    assert torch.equal(out, U.FP8LinearFunctionBase.fp8_mlp_fwd(x.detach(), mlp.w1, mlp.w2)[3])
    do3 = bf((M, H), seed=12)
    out.backward(do3)
    xr = x.detach().double().requires_grad_(True)
    w1, w2 = mlp.w1.detach().double().requires_grad_(True), mlp.w2.detach().double().requires_grad_(True)
    o1 = xr @ w1
    ref = (torch.nn.functional.silu(o1[:, :I]) * o1[:, I:]) @ w2
    ref.backward(do3.double())
    assert rel(out, ref.detach()) < FP8_REL2
    assert rel(x.grad, xr.grad) < FP8_REL3
    assert rel(mlp.w1.main_grad, w1.grad) < FP8_REL3 and rel(mlp.w2.main_grad, w2.grad) < FP8_REL3
    # the functional backward returns the same dx and dW2; its dW1 uses x quantised once, while the
    # autograd function re-quantises the dequantised FP8 copy it saved (fp8_utils.py:781-792)
    dx, dw1, dw2 = U.FP8LinearFunctionBase.fp8_mlp_bwd(do3, x.detach(), mlp.w1.detach(), mlp.w2.detach())
    assert rel(dx, x.grad) < 1e-2 and rel(dw2, mlp.w2.main_grad) < 1e-2 and rel(dw1, mlp.w1.main_grad) < FP8_REL


def test_fused_norm_fp8_mlp(U):
    from paddleformers_amd import functional as F8

    H, I, B, S = 512, 256, 2, 256
    norm_w = torch.nn.Parameter((bf((H,), 0.1, seed=13).float() + 1).to(torch.bfloat16))
    mlp = U.FP8Mlp(H, I, device="cuda", using_post_norm_recompute=True, norm_weight=norm_w, norm_eps=1e-6)
    with torch.no_grad():
        mlp.w1.copy_(bf((H, 2 * I), 0.05, seed=14))
        mlp.w2.copy_(bf((I, H), 0.05, seed=15))
    x = bf((B, S, H), seed=16).requires_grad_(True)
    out = mlp(x)
    assert out.shape == (B, S, H)
    # forward == norm followed by the plain FP8 MLP, bit for bit
    y, _ = F8.fused_rms_norm_ext(x.detach(), norm_w.detach(), 1e-6)
    assert torch.equal(out.reshape(-1, H), U.FP8LinearFunctionBase.fp8_mlp_fwd(y.reshape(-1, H), mlp.w1, mlp.w2)[3])
    assert torch.equal(out, U.FP8LinearFunctionBase.fp8_mlp_fwd_norm_rc(x.detach(), norm_w.detach(), 1e-6, mlp.w1, mlp.w2))
    do3 = bf((B, S, H), seed=17)
    out.backward(do3)
    xr = x.detach().double().requires_grad_(True)
    nw = norm_w.detach().double().requires_grad_(True)
    w1, w2 = mlp.w1.detach().double().requires_grad_(True), mlp.w2.detach().double().requires_grad_(True)
    yn = xr * torch.rsqrt((xr * xr).mean(dim=-1, keepdim=True) + 1e-6) * nw
    o1 = yn @ w1
    ref = (torch.nn.functional.silu(o1[..., :I]) * o1[..., I:]) @ w2
    ref.backward(do3.double())
    assert rel(out, ref.detach()) < FP8_REL2
    assert rel(x.grad, xr.grad) < FP8_REL3
    assert rel(norm_w.grad, nw.grad) < FP8_REL3
    assert rel(mlp.w1.grad, w1.grad) < FP8_REL3 and rel(mlp.w2.grad, w2.grad) < FP8_REL3
    # the recompute-style functional backward: same dx, gradients accumulated on the parameters
    norm_w2 = norm_w.detach().clone()
    norm_w2.main_grad = None
    w1b, w2b = mlp.w1.detach().clone(), mlp.w2.detach().clone()
    w1b.main_grad = None
    w2b.main_grad = None
    dx, norm_out, invar = U.FP8LinearFunctionBase.fp8_mlp_bwd_norm_rc(do3, x.detach(), norm_w2, 1e-6, w1b, w2b)
    assert rel(dx, x.grad) < 1e-2 and rel(norm_w2.main_grad, norm_w.grad) < 2e-2 and rel(w1b.main_grad, mlp.w1.grad) < 2e-2
