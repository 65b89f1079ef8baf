"""The Paddle binding shipped as paddleformers_amd/paddle_backend.py, executed as written.

Paddle is not installed, so the dozen `paddle.*` names the binding uses (dtypes, `empty`, the stream accessor, the
`incubate.nn.functional` namespace, `Tensor.strides` / `Tensor.astype`) are provided here on top of torch tensors.  What this
pins is the C side of every call in that text: argument order, layout flags, output shapes.  Every function is compared
byte for byte with the package's own binding of the same entry point.
"""
from __future__ import annotations

import os
import sys
import types

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from paddleformers_amd import _lib as L
from paddleformers_amd import deep_gemm as D
from paddleformers_amd import functional as F

from . import _gen as G

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _fake_paddle():
    p = types.ModuleType("paddle")
    p.float8_e4m3fn, p.float32, p.bfloat16, p.uint8, p.int32 = (torch.float8_e4m3fn, torch.float32, torch.bfloat16,
                                                                 torch.uint8, torch.int32)
    p.empty = lambda shape, dtype=None: torch.empty(tuple(int(v) for v in shape), dtype=dtype, device="cuda")

    class _Base:
        @property
        def raw_stream(self):
            return torch.cuda.current_stream().cuda_stream

    class _Stream:
        stream_base = _Base()

    p.device = types.SimpleNamespace(current_stream=lambda: _Stream())
    p.incubate = types.SimpleNamespace(nn=types.SimpleNamespace(functional=types.SimpleNamespace()))
    return p


@pytest.fixture(scope="module")
def stub():
    code = open(os.path.join(ROOT, "paddleformers_amd", "paddle_backend.py")).read()
    assert "..." not in code, "the binding must be written out in full"
    assert 'ctypes.CDLL("libpf8.so")' in code
    code = code.replace('ctypes.CDLL("libpf8.so")', f"ctypes.CDLL({L.LIB_PATH!r})")   # the in-tree build, by path
    L.lib()                                                                          # raises if the library is missing
    saved = {n: sys.modules.get(n) for n in ("paddle", "paddlefleet_ops")}
    had = {n: hasattr(torch.Tensor, n) for n in ("strides", "astype")}
    torch.Tensor.strides = property(lambda self: list(self.stride()))
    torch.Tensor.astype = lambda self, dt: self.to(dt)
    sys.modules["paddle"] = _fake_paddle()
    ns = {"__name__": "pf8_backend"}
    try:
        exec(compile(code, "paddle_backend.py", "exec"), ns)
        ns["install"]()
        yield types.SimpleNamespace(**ns)
    finally:
        for n, m in saved.items():
            if m is None:
                sys.modules.pop(n, None)
            else:
                sys.modules[n] = m
        for n, h in had.items():
            if not h:
                delattr(torch.Tensor, n)


def _same(a, b):
    if isinstance(a, (tuple, list)):
        assert len(a) == len(b)
        for x, y in zip(a, b):
            _same(x, y)
        return
    assert tuple(a.shape) == tuple(b.shape) and a.dtype == b.dtype
    wa = a.contiguous().view(torch.uint8) if a.numel() else a
    wb = b.contiguous().view(torch.uint8) if b.numel() else b
    assert torch.equal(wa, wb)


def _x(shape, seed):
    return G.to_torch_bf16(G.bf16_normal(shape, seed, std=1.0, outlier_frac=0.01, outlier_scale=30.0))


def test_install_binds_every_operator_of_the_path(stub):
    ops = sys.modules["paddlefleet_ops"]
    for name in ("fp8_gemm_nt", "m_grouped_fp8_gemm_nt_contiguous", "m_grouped_fp8_gemm_nt_masked", "set_num_sms"):
        assert callable(getattr(ops.deep_gemm, name))
    fn = sys.modules["paddle"].incubate.nn.functional
    for name in ("fp8_quant_blockwise", "fused_stack_transpose_quant", "fused_weighted_swiglu_act_quant",
                 "fused_transpose_split_quant", "fused_act_dequant", "fused_swiglu_weighted_bwd", "fp8_gemm_blockwise"):
        assert callable(getattr(fn, name))


@pytest.mark.parametrize("kw", [
    dict(quant_method="1x128"),
    dict(quant_method="1x128", output_scale_transpose=True, using_pow2_scale=True),
    dict(quant_method="1x128", input_transpose=True, output_scale_transpose=True),
    dict(quant_method="1x128", input_transpose=True, output_scale_transpose=False),
    dict(quant_method="1x128", input_transpose=True, output_scale_transpose=True, return_transpose_only=True),
    dict(quant_method="128x128", output_scale_transpose=False, input_transpose=False, return_transpose_only=False),
    dict(quant_method="128x128", output_scale_transpose=False, input_transpose=True, return_transpose_only=True),
    dict(quant_method="128x128", output_scale_transpose=False, input_transpose=True, return_transpose_only=False),
])
def test_fp8_quant_blockwise_every_keyword_combination_of_the_reference(stub, kw):
    x = _x((384, 512), 11)
    _same(stub.fp8_quant_blockwise(x, **kw), F.fp8_quant_blockwise(x, **kw))


def test_quantizers_and_activation_operators(stub):
    ws = [_x((256, 384), 20 + i) for i in range(3)]
    for tr in (False, True):
        _same(stub.fused_stack_transpose_quant(ws, transpose=tr), F.fused_stack_transpose_quant(ws, transpose=tr))
    o1 = _x((384, 512), 31)
    probs = torch.rand(384, 1, device="cuda")
    for pow2 in (False, True):
        _same(stub.fused_weighted_swiglu_act_quant(o1, probs, using_pow2_scaling=pow2),
              F.fused_weighted_swiglu_act_quant(o1, probs, using_pow2_scaling=pow2))
    _same(stub.fused_weighted_swiglu_act_quant(o1), F.fused_weighted_swiglu_act_quant(o1))
    do2 = _x((384, 256), 32)
    _same(stub.fused_swiglu_weighted_bwd(o1, do2, probs), F.fused_swiglu_weighted_bwd(o1, do2, probs))

    rows = [128, 0, 256]
    x = _x((384, 256), 33)
    _same(stub.fused_transpose_split_quant(x, None, rows, True), F.fused_transpose_split_quant(x, None, rows, True))
    q, s = F.fp8_quant_blockwise(x, quant_method="1x128", output_scale_transpose=True)   # the node's cached input: s.T
    _same(stub.fused_transpose_split_quant(q, s.T, rows, False), F.fused_transpose_split_quant(q, s.T, rows, False))
    _same(stub.fused_act_dequant(q, s.T), F.fused_act_dequant(q, s.T))
    q0, s0 = F.fp8_quant_blockwise(x, quant_method="1x128")
    _same(stub.fused_act_dequant(q0, s0), F.fused_act_dequant(q0, s0))


def test_weight_gradient_gemm(stub):
    a, b = _x((256, 384), 41), _x((256, 512), 42)                       # [tokens, Ka], [tokens, Nb]
    (qa,), (sa,) = F.fused_transpose_split_quant(a, None, [256], True)
    (qb,), (sb,) = F.fused_transpose_split_quant(b, None, [256], True)
    ref = F.fp8_gemm_blockwise(a=qa, a_decode_scale=sa, b=qb, b_decode_scale=sb, out_dtype=torch.float32)
    got = stub.fp8_gemm_blockwise(a=qa, a_decode_scale=sa, b=qb, b_decode_scale=sb, out_dtype=torch.float32, out=None,
                                  accumulate=False, use_split_accumulator=True, is_a_1d_scaled=True, is_b_1d_scaled=True)
    _same(got, ref)
    acc_ref, acc_got = ref.clone(), ref.clone()
    F.fp8_gemm_blockwise(a=qa, a_decode_scale=sa, b=qb, b_decode_scale=sb, out=acc_ref, accumulate=True)
    stub.fp8_gemm_blockwise(a=qa, a_decode_scale=sa, b=qb, b_decode_scale=sb, out_dtype=torch.float32, out=acc_got, accumulate=True)
    _same(acc_got, acc_ref)
    # the (1, 1, 128) recipe of deep_gemm.fp8_gemm_nt is the same kernel: scales arrive as `.t()` views
    o_ref = torch.empty(384, 512, dtype=torch.float32, device="cuda")
    o_got = torch.empty_like(o_ref)
    D.fp8_gemm_nt((qa, sa.t()), (qb, sb.t()), o_ref, recipe=(1, 1, 128))
    stub.deep_gemm.fp8_gemm_nt((qa, sa.t()), (qb, sb.t()), o_got, c=None, recipe=(1, 1, 128), compiled_dims="mn")
    _same(o_got, o_ref)


@pytest.mark.parametrize("ue8m0", [False, True])
def test_dense_and_grouped_gemms(stub, ue8m0):
    M, N, K, E = 512, 512, 512, 3
    x = _x((M, K), 51)
    q, s = F.fp8_quant_blockwise(x, quant_method="1x128", output_scale_transpose=True, using_pow2_scale=ue8m0)
    w = [_x((K, N), 60 + e) for e in range(E)]
    wq, ws = F.fused_stack_transpose_quant(w, transpose=True, using_pow2_scale=ue8m0)
    wq, ws = wq.view(E, N, K), ws.view(E, N // 128, K // 128)
    if ue8m0:
        s, ws = F.scales_to_ue8m0(s), F.scales_to_ue8m0(ws)
    ref = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    got = torch.empty_like(ref)
    D.fp8_gemm_nt((q, s.T), (wq[0], ws[0]), ref)
    stub.deep_gemm.fp8_gemm_nt((q, s.T), (wq[0], ws[0]), got)
    _same(got, ref)
    m_idx = torch.tensor(np.repeat([0, 2, -1, 1], 128), dtype=torch.int32, device="cuda")
    ref.zero_()
    got.zero_()
    D.m_grouped_fp8_gemm_nt_contiguous((q, s.T), (wq, ws), ref, m_indices=m_idx)
    stub.deep_gemm.m_grouped_fp8_gemm_nt_contiguous((q, s.T), (wq, ws), got, m_indices=m_idx)
    _same(got, ref)


def test_masked_gemm_and_the_compute_unit_budget(stub):
    E, Mmax, N, K = 3, 256, 256, 384
    x = _x((E * Mmax, K), 71)
    q, s = F.fp8_quant_blockwise(x, quant_method="1x128")
    w = [_x((K, N), 80 + e) for e in range(E)]
    wq, ws = F.fused_stack_transpose_quant(w, transpose=True)
    a = (q.view(E, Mmax, K), s.view(E, Mmax, K // 128))
    b = (wq.view(E, N, K), ws.view(E, N // 128, K // 128))
    masked = torch.tensor([200, 0, 256], dtype=torch.int32, device="cuda")
    ref = torch.zeros(E, Mmax, N, dtype=torch.bfloat16, device="cuda")
    got = torch.zeros_like(ref)
    D.m_grouped_fp8_gemm_nt_masked(a, b, ref, masked, 128)
    stub.deep_gemm.m_grouped_fp8_gemm_nt_masked(a, b, got, masked, 128)
    _same(got, ref)
    before = D.get_num_sms()
    try:
        stub.deep_gemm.set_num_sms(24)
        assert D.get_num_sms() == 24 and stub.deep_gemm.get_num_sms() == 24
    finally:
        D.set_num_sms(before)
