"""GPU tests of the ERNIE dense FP8 SwiGLU MLP wrappers (Fp8FusedMlpFunc, MemEfficientFp8FusedMlpFunc,
Fp8FusedMlp, fp8_gemm, padding): against float64 autograd within FP8 tolerances, against the
already-verified building blocks for exact consistency, and for the reference's padding rule."""
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

FP8_REL = 0.06      # one FP8 GEMM stage against exact math
FP8_REL2 = 0.10     # two chained stages
FP8_REL3 = 0.15     # three


def rel(a, b):
    a, b = a.detach().double(), b.detach().double()
    return float(((a - b).norm() / (b.norm() + 1e-30)).detach())


def bf(shape, std=1.0, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, device="cuda", generator=g) * std).to(torch.bfloat16)


@pytest.fixture(scope="module")
def EL():
    from paddleformers_amd import _lib
    from paddleformers_amd import ernie_fp8_linear

    _lib.lib()
    return ernie_fp8_linear


@pytest.mark.parametrize("n", [512, 1024, 100, 384, 130, 600, 900])
def test_padding_goes_to_the_next_multiple_of_512(EL, n):
    # the reference picks a step of 128 or 512 from the size; worked out by hand for these sizes, both
    # branches end on the next multiple of 512
    want = -(-n // 512) * 512
    x = torch.ones((n, 8), dtype=torch.bfloat16, device="cuda")
    out = EL.padding(x, 0)
    assert out.shape == (want, 8) and torch.equal(out[:n], x) and not out[n:].any()
    out1 = EL.padding(x.t().contiguous(), 1)
    assert out1.shape == (8, want) and not out1[:, n:].any()


class _Cfg:
    hidden_size, intermediate_size = 512, 256


@pytest.mark.parametrize("func", ["plain", "mem_efficient"])
@pytest.mark.parametrize("shape", [(512,), (2, 150)])
def test_fused_mlp_forward_backward(EL, func, shape):
    from paddleformers_amd import fp8_utils as U

    H, I = _Cfg.hidden_size, _Cfg.intermediate_size
    mlp = EL.Fp8FusedMlp(_Cfg())
    with torch.no_grad():
        mlp.w1.copy_(bf((H, 2 * I), 0.05, seed=9))
        mlp.w2.copy_(bf((I, H), 0.05, seed=10))
    x = bf((*shape, H), seed=11).requires_grad_(True)
    fn = EL.Fp8FusedMlpFunc if func == "plain" else EL.MemEfficientFp8FusedMlpFunc
    out = fn.apply(x, mlp.w1, mlp.w2)
    assert out.shape == (*shape, H) if len(shape) == 1 else out.shape == (shape[0], shape[1], H)
    # same arithmetic as the transformers wrapper's forward: identical output
    ref_fwd = U.FP8LinearFunctionBase.fp8_mlp_fwd(x.detach().reshape(-1, H), mlp.w1.detach(), mlp.w2.detach())[3]
    assert torch.equal(out.reshape(-1, H), ref_fwd)
    if func == "plain":
        assert torch.equal(mlp(x), out)
    do3 = bf((*shape, H), seed=12)
    out.backward(do3)
    xr = x.detach().double().requires_grad_(True)
    w1, w2 = mlp.w1.detach().double().requires_grad_(True), mlp.w2.detach().double().requires_grad_(True)
    o1 = xr @ w1
    ref = (torch.nn.functional.silu(o1[..., :I]) * o1[..., I:]) @ w2
    ref.backward(do3.double())
    assert rel(out, ref) < FP8_REL2
    assert x.grad.shape == x.shape and rel(x.grad, xr.grad) < FP8_REL3
    assert mlp.w1.grad.dtype == torch.bfloat16 and rel(mlp.w1.grad, w1.grad) < FP8_REL3
    assert rel(mlp.w2.grad, w2.grad) < FP8_REL3


def test_the_two_functions_agree(EL):
    H, I, M = 512, 256, 300
    w1, w2 = bf((H, 2 * I), 0.05, seed=1).requires_grad_(True), bf((I, H), 0.05, seed=2).requires_grad_(True)
    x, do3 = bf((M, H), seed=3), bf((M, H), seed=4)
    grads = []
    for fn in (EL.Fp8FusedMlpFunc, EL.MemEfficientFp8FusedMlpFunc):
        xi = x.clone().requires_grad_(True)
        w1.grad = w2.grad = None
        out = fn.apply(xi, w1, w2)
        out.backward(do3)
        grads.append((out.detach(), xi.grad, w1.grad.clone(), w2.grad.clone()))
    a, b = grads
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]) and torch.equal(a[3], b[3])
    # dW1: the memory-saving variant transposes the dequantized FP8 input instead of the input itself
    assert rel(a[2], b[2]) < FP8_REL


def test_fp8_gemm_forms(EL):
    from paddleformers_amd import functional as F8

    M, Ka, Nb = 256, 384, 128
    a, b = bf((M, Ka), seed=5), bf((M, Nb), seed=6)
    a_t, sa_t = F8.fp8_quant_blockwise(a, quant_method="1x128", input_transpose=True, output_scale_transpose=True, return_transpose_only=True)
    b_t, sb_t = F8.fp8_quant_blockwise(b, quant_method="1x128", input_transpose=True, output_scale_transpose=True, return_transpose_only=True)
    y = EL.fp8_gemm(a_t, sa_t, b_t, sb_t, True, True, rtn_dtype=torch.float32)
    assert y.dtype == torch.float32 and y.shape == (Ka, Nb)
    assert rel(y, a.double().t() @ b.double()) < FP8_REL
    acc = y.clone()
    out = EL.fp8_gemm(a_t, sa_t, b_t, sb_t, True, True, out=acc)
    assert out is acc and rel(acc, 2 * y) < 1e-6
    # zero-sized operands: zeros, or `out` unchanged
    z = EL.fp8_gemm(a_t[:0], sa_t[:, :0], b_t, sb_t, True, True, rtn_dtype=torch.float32)
    assert z.shape == (0, Nb)
    # 128x128-scaled second operand: the forward GEMM (scales handed over transposed)
    xq, xs = F8.fp8_quant_blockwise(a, quant_method="1x128", input_transpose=False, output_scale_transpose=True)
    w = bf((Ka, 256), 0.05, seed=7)
    wq, ws = F8.fp8_quant_blockwise(w, quant_method="128x128", input_transpose=True, output_scale_transpose=False, return_transpose_only=True)
    c = EL.fp8_gemm(xq, xs, wq, ws.t().contiguous(), True, False)
    assert c.dtype == torch.bfloat16 and rel(c, a.double() @ w.double()) < FP8_REL
    with pytest.raises(ValueError):
        EL.fp8_gemm(xq, xs, wq, ws.t().contiguous(), True, False, out=c)
