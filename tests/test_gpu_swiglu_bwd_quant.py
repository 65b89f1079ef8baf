"""GPU tests of the SwiGLU backward that writes its results in quantized form only, through the C ABI.

The reference runs the SwiGLU backward (transformers/fp8_utils.py:1049-1052) and then quantizes do1 row-wise for the dgrad
GEMM (:1073-1079) and, per expert and transposed, do1 (:1168) and o2_s (:1115) for the two weight gradients.  The one
kernel must give the bytes and scales of that chain: checked against the oracle's chain (SwiGLU backward, 1x128
quantization, per-expert transposed quantization) and against the library's own separate entry points.  probs_grad is a
sum taken in another order, held to 1e-5 of the sum of the magnitudes of its terms."""
import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

PG_TOL = 1e-5      # |probs_grad - oracle| <= PG_TOL * sum_j |do2_s[j] * o2[j]| per row


def _inputs(I, rows, seed):
    M = sum(rows)
    o1 = G.bf16_normal((M, 2 * I), seed=seed, std=2.0, outlier_frac=1e-3, outlier_scale=20.0)
    do2 = G.bf16_normal((M, I), seed=seed + 1, std=0.5, outlier_frac=1e-3, outlier_scale=50.0)
    probs = np.random.default_rng(seed + 2).uniform(0.05, 0.95, M).astype(np.float32)
    return o1, do2, probs


def _u8(t):
    return t.view(torch.uint8) if t.dtype == torch.float8_e4m3fn else t


@pytest.mark.parametrize("I,rows,pow2_rows,ue8m0,pow2_t", [
    (128, [128], False, False, True),
    (256, [256, 0, 128, 384], True, False, True),
    (384, [128] * 5 + [0, 640], True, True, True),
    (1408, [512, 0, 1024, 128], True, True, True),
    (256, [384, 128], False, False, False),          # exact scales (amax / 448) in both directions
    (384, [256, 256], True, False, False),
])
def test_quantized_forms_equal_the_chain_of_separate_operators(I, rows, pow2_rows, ue8m0, pow2_t):
    from paddleformers_amd import functional as F8

    o1, do2, probs = _inputs(I, rows, seed=7 * I + len(rows))
    M = sum(rows)
    to1, tdo2, tp = G.to_torch_bf16(o1), G.to_torch_bf16(do2), torch.from_numpy(probs).cuda()
    q, s, qt, st, oqt, ost, pg = F8.swiglu_weighted_bwd_quant(to1, tdo2, tp, rows, pow2_rows, pow2_t, ue8m0)
    # the oracle's chain
    edo1, epg, eo2s = O.swiglu_weighted_bwd(o1, do2, probs)
    eq, es = O.quant_1x128(edo1, 1, pow2=pow2_rows)
    assert not G.mismatch_report(G.from_torch_fp8(q), eq, "do1 row-wise bytes")
    if ue8m0:
        assert s.dtype == torch.uint8 and np.array_equal(s.cpu().numpy(), (es.view(np.uint32) >> 23).astype(np.uint8))
    else:
        assert np.array_equal(s.cpu().numpy().view(np.uint32), es.view(np.uint32))
    for name, got_q, got_s, src, K in (("do1", qt, st, edo1, 2 * I), ("o2_s", oqt, ost, eo2s, I)):
        eqs, ess = O.transpose_split_quant(src, None, rows, pow2_t)
        for e, r in enumerate(rows):
            assert tuple(got_q[e].shape) == (K, r) and tuple(got_s[e].shape) == (r // 128, K)
            if r:
                assert not G.mismatch_report(G.from_torch_fp8(got_q[e]), eqs[e], f"{name}^T bytes, expert {e}")
                assert np.array_equal(got_s[e].cpu().numpy().view(np.uint32), ess[e].view(np.uint32)), f"{name}^T scales, expert {e}"
    o2 = O.bf16_bits_to_f32(eo2s) / probs[:, None]
    terms = np.abs(O.bf16_bits_to_f32(do2) * o2).sum(axis=1)
    assert np.all(np.abs(pg.cpu().numpy() - epg) <= PG_TOL * terms + 1e-30)
    # the library's own chain
    do1, pg0, o2s = F8.fused_swiglu_weighted_bwd(to1, tdo2, tp)
    q0, s0, qt0, st0 = F8.quant_and_transpose_split(do1, rows, pow2_rows, pow2_t, ue8m0_scale=ue8m0)
    oqt0, ost0 = F8.fused_transpose_split_quant(o2s, None, rows, pow2_t)
    assert torch.equal(_u8(q), _u8(q0)) and torch.equal(s, s0)
    for a, b in ((qt, qt0), (st, st0), (oqt, oqt0), (ost, ost0)):
        assert torch.equal(_u8(a.buf), _u8(b.buf))
    assert np.all(np.abs((pg - pg0).cpu().numpy()) <= PG_TOL * terms + 1e-30)
    assert M == 0 or float(pg.abs().max()) > 0


def test_row_scales_in_either_layout():
    from paddleformers_amd import functional as F8

    I, rows = 256, [128, 0, 384]
    o1, do2, probs = _inputs(I, rows, seed=9)
    args = (G.to_torch_bf16(o1), G.to_torch_bf16(do2), torch.from_numpy(probs).cuda(), rows)
    for pow2 in (False, True):
        a = F8.swiglu_weighted_bwd_quant(*args, pow2, True)
        b = F8.swiglu_weighted_bwd_quant(*args, pow2, True, output_scale_transpose=False)
        assert tuple(b[1].shape) == (sum(rows), 2 * I // 128) and torch.equal(b[1], a[1].t().contiguous())
        for x, y in zip(a[:1] + a[2:6], b[:1] + b[2:6]):
            assert torch.equal(_u8(getattr(x, "buf", x)), _u8(getattr(y, "buf", y)))
        assert torch.equal(a[6], b[6])
    with pytest.raises(ValueError):
        F8.swiglu_weighted_bwd_quant(*args, True, True, True, output_scale_transpose=False)


def test_probs_grad_does_not_depend_on_how_rows_are_grouped_into_experts():
    """A row's sum is taken over its own 128-column tiles in their order, whatever tile the row sits in."""
    from paddleformers_amd import functional as F8

    I = 384
    o1, do2, probs = _inputs(I, [768], seed=5)
    args = (G.to_torch_bf16(o1), G.to_torch_bf16(do2), torch.from_numpy(probs).cuda())
    a = F8.swiglu_weighted_bwd_quant(*args, [768], True, True)
    b = F8.swiglu_weighted_bwd_quant(*args, [128, 256, 0, 384], True, True)
    assert torch.equal(a[6], b[6]) and torch.equal(_u8(a[0]), _u8(b[0])) and torch.equal(a[1], b[1])


def test_rejects_bad_input_and_takes_empty_input():
    from paddleformers_amd import functional as F8

    o1 = torch.zeros((256, 512), dtype=torch.bfloat16, device="cuda")
    do2 = torch.zeros((256, 256), dtype=torch.bfloat16, device="cuda")
    p = torch.ones(256, device="cuda")
    with pytest.raises(ValueError):
        F8.swiglu_weighted_bwd_quant(o1, do2, p, [128, 64, 64])
    with pytest.raises(ValueError):
        F8.swiglu_weighted_bwd_quant(o1, do2, p, [128])
    with pytest.raises(ValueError):
        F8.swiglu_weighted_bwd_quant(o1, do2[:, :128], p, [256])
    with pytest.raises(ValueError):
        F8.swiglu_weighted_bwd_quant(o1[:, :384], do2[:, :192], p, [256])       # I = 192 is not a multiple of 128
    with pytest.raises(ValueError):
        F8.swiglu_weighted_bwd_quant(o1, do2, p, [256], False, True, True)      # exponent bytes need power-of-two scales
    out = F8.swiglu_weighted_bwd_quant(o1[:0], do2[:0], p[:0], [0, 0], True, True)
    assert tuple(out[0].shape) == (0, 512) and len(out[2]) == 2 and out[6].numel() == 0
    # zero rows (the padding of an expert's segment) quantize to zero bytes with scale 1 and a zero probs_grad
    q, s, qt, st, oqt, ost, pg = F8.swiglu_weighted_bwd_quant(o1, do2, p, [256], True, True)
    assert not _u8(q).any() and not pg.any() and bool((s == 1).all()) and bool((st.buf == 1).all())


def test_c_abi_argument_checks():
    import ctypes as C

    from paddleformers_amd import _lib

    L = _lib.lib()
    rows = (C.c_int64 * 1)(100)
    z = C.c_void_p(0)
    rc = L.pf8_swiglu_weighted_bwd_quant(z, z, z, rows, 1, 128, z, z, 1, 0, z, z, z, z, 1, z, z, z)
    assert rc != 0 and b"multiples of 128" in L.pf8_last_error()
    rows = (C.c_int64 * 1)(128)
    rc = L.pf8_swiglu_weighted_bwd_quant(z, z, z, rows, 1, 128, z, z, 1, 0, z, z, z, z, 1, z, z, z)
    assert rc != 0 and b"null pointer" in L.pf8_last_error()
    rc = L.pf8_swiglu_weighted_bwd_quant(z, z, z, rows, 1, 100, z, z, 1, 0, z, z, z, z, 1, z, z, z)
    assert rc != 0 and b"multiple of 128" in L.pf8_last_error()
