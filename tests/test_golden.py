"""Committed golden fixtures (tests/golden/pf8_golden.npz, written by tests/golden/make_fixtures.py):
without a GPU, the CPU oracle must reproduce every stored output to the bit; with one, the HIP path is
checked against the same stored data through the reference-named host mirror (bytes, scales and elementwise
results bit-exact; GEMM outputs within 1e-3 relative Frobenius error, the bar of the path)."""
import importlib.util
import os

import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden", "pf8_golden.npz")
GEMM_FRO = 1e-3


@pytest.fixture(scope="module")
def gold():
    with np.load(GOLDEN, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32) if a.dtype == np.float32 else a


def test_the_oracle_reproduces_every_fixture(gold):
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    fresh = mod.build()
    assert sorted(fresh) == sorted(gold)
    for k in sorted(gold):
        assert fresh[k].dtype == gold[k].dtype and fresh[k].shape == gold[k].shape, k
        assert np.array_equal(_bits(fresh[k]), _bits(gold[k])), f"{k}: {np.count_nonzero(_bits(fresh[k]) != _bits(gold[k]))} elements differ"


def _same(got, exp, what):
    got, exp = _bits(np.asarray(got)), _bits(exp)
    assert got.shape == exp.shape, f"{what}: shape {got.shape} vs {exp.shape}"
    assert np.array_equal(got, exp), f"{what}: {np.count_nonzero(got != exp)} of {exp.size} differ"


@pytest.mark.gpu
def test_quantizers_match_the_fixtures(gold):
    torch = pytest.importorskip("torch")
    from paddleformers_amd import functional as F

    x = G.to_torch_bf16(gold["act_x"])
    for pow2 in (0, 1):
        q, s = F.fp8_quant_blockwise(x, quant_method="1x128", using_pow2_scale=bool(pow2))
        _same(G.from_torch_fp8(q), gold[f"quant_1x128_p{pow2}_q"], f"1x128 bytes pow2={pow2}")
        _same(s.cpu().numpy(), gold[f"quant_1x128_p{pow2}_s"], f"1x128 scales pow2={pow2}")
    _, s = F.fp8_quant_blockwise(x, quant_method="1x128", output_scale_transpose=True)
    _same(s.cpu().numpy(), gold["quant_1x128_layout1_s"], "1x128 transposed scales")
    q, s, qt, st = F.fp8_quant_blockwise(x, quant_method="1x128", input_transpose=True, output_scale_transpose=True)
    _same(G.from_torch_fp8(q), gold["quant_transpose_q"], "quant+transpose bytes")
    _same(s.cpu().numpy(), gold["quant_transpose_s"], "quant+transpose scales")
    _same(G.from_torch_fp8(qt), gold["quant_transpose_qt"], "quant+transpose transposed bytes")
    _same(st.cpu().numpy(), gold["quant_transpose_st"], "quant+transpose transposed scales")
    w, w2 = G.to_torch_bf16(gold["weight_w"]), G.to_torch_bf16(gold["weight_w2"])
    q, s, qt, st = F.fp8_quant_blockwise(w, quant_method="128x128", input_transpose=True)
    for got, key in ((q, "q"), (qt, "qt")):
        _same(G.from_torch_fp8(got), gold[f"quant_128x128_{key}"], f"128x128 {key}")
    for got, key in ((s, "s"), (st, "st")):
        _same(got.cpu().numpy(), gold[f"quant_128x128_{key}"], f"128x128 {key}")
    for tr in (0, 1):
        q, s = F.fused_stack_transpose_quant([w, w2], transpose=bool(tr))
        _same(G.from_torch_fp8(q), gold[f"stack_quant_t{tr}_q"], f"stack quant bytes t={tr}")
        _same(s.cpu().numpy(), gold[f"stack_quant_t{tr}_s"], f"stack quant scales t={tr}")
    o1, probs = G.to_torch_bf16(gold["swiglu_o1"]), torch.from_numpy(gold["swiglu_probs"]).cuda()
    for pow2 in (0, 1):
        q, s, o2 = F.fused_weighted_swiglu_act_quant(o1, probs, using_pow2_scaling=bool(pow2), return_o2=True)
        _same(G.from_torch_fp8(q), gold[f"swiglu_quant_p{pow2}_q"], f"swiglu bytes pow2={pow2}")
        _same(s.cpu().numpy(), gold[f"swiglu_quant_p{pow2}_s"], f"swiglu scales pow2={pow2}")
        _same(G.from_torch_bf16(o2), gold["swiglu_quant_o2"], "swiglu activations")
    do1, pg, o2s = F.fused_swiglu_weighted_bwd(o1, G.to_torch_bf16(gold["swiglu_bwd_do2"]), probs)
    _same(G.from_torch_bf16(do1), gold["swiglu_bwd_do1"], "swiglu backward do1")
    # a row sum of 256 fp32 products: the summation order is the kernel's own
    assert np.allclose(pg.cpu().numpy(), gold["swiglu_bwd_pg"], rtol=1e-5, atol=1e-7)
    _same(G.from_torch_bf16(o2s), gold["swiglu_bwd_o2s"], "swiglu backward o2_s")
    # the backward that writes quantized forms only: the quantizations of the golden do1 and o2_s
    fq, fs, fqt, fst, foqt, fost, fpg = F.swiglu_weighted_bwd_quant(o1, G.to_torch_bf16(gold["swiglu_bwd_do2"]), probs, [128], False, True)
    eq, es = O.quant_1x128(gold["swiglu_bwd_do1"], 1)
    _same(G.from_torch_fp8(fq), eq, "fused swiglu backward: do1 bytes")
    _same(fs.cpu().numpy(), es, "fused swiglu backward: do1 scales")
    for got_q, got_s, key in ((fqt, fst, "swiglu_bwd_do1"), (foqt, fost, "swiglu_bwd_o2s")):
        etq, ets = O.transpose_split_quant(gold[key], None, [128], True)
        _same(G.from_torch_fp8(got_q[0]), etq[0], f"fused swiglu backward: {key} transposed bytes")
        _same(got_s[0].cpu().numpy(), ets[0], f"fused swiglu backward: {key} transposed scales")
    assert np.allclose(fpg.cpu().numpy(), gold["swiglu_bwd_pg"], rtol=1e-5, atol=1e-7)
    rows = [int(r) for r in gold["split_rows"]]
    xs3 = G.to_torch_bf16(gold["split_x"])
    qs, ss = F.fused_transpose_split_quant(xs3, None, rows, True)
    xq, xsc = F.fp8_quant_blockwise(xs3, quant_method="1x128")
    qf, sf = F.fused_transpose_split_quant(xq, xsc, rows, True)
    for e in (0, 2):
        _same(G.from_torch_fp8(qs[e]), gold[f"split_bf16_q{e}"], f"split quant bytes expert {e}")
        _same(ss[e].cpu().numpy(), gold[f"split_bf16_s{e}"], f"split quant scales expert {e}")
        _same(G.from_torch_fp8(qf[e]), gold[f"split_fp8_q{e}"], f"split quant (e4m3 source) bytes expert {e}")
        _same(sf[e].cpu().numpy(), gold[f"split_fp8_s{e}"], f"split quant (e4m3 source) scales expert {e}")


def _same_but_nan(got_bits, exp_bits, what):
    nan_e, nan_g = (exp_bits & 0x7FFF) > 0x7F80, (got_bits & 0x7FFF) > 0x7F80
    assert np.array_equal(nan_e, nan_g), f"{what}: NaN positions differ"
    assert np.array_equal(got_bits[~nan_e], exp_bits[~nan_e]), f"{what}: values differ"


@pytest.mark.gpu
def test_dequantizers_match_the_fixtures(gold):
    torch = pytest.importorskip("torch")
    from paddleformers_amd import checkpoint_dequant as CD
    from paddleformers_amd import functional as F

    out = F.fused_act_dequant(G.to_torch_fp8(gold["quant_1x128_p0_q"]), torch.from_numpy(gold["quant_1x128_p0_s"]).cuda())
    _same(G.from_torch_bf16(out), gold["act_dequant_out"], "1x128 dequant")
    q = G.to_torch_fp8(gold["weight_dequant_q"])                   # random codes: both NaN codes occur
    out = F.weight_dequant(q, torch.from_numpy(gold["weight_dequant_s"]).cuda())
    _same_but_nan(G.from_torch_bf16(out), gold["weight_dequant_out"], "128x128 dequant")
    dq = CD.get_checkpoint_dequantizer("fp8_block").configure_formats("e4m3", "ue8m0").configure_geometry((0, 1), (128, 128))
    out = dq.dequantize({"qweight": q.view(torch.uint8), "scale": torch.from_numpy(gold["block_dequant_e8"]).cuda()}, torch.bfloat16)
    _same_but_nan(G.from_torch_bf16(out), gold["block_dequant_out"], "block dequant, UE8M0 scales")
    e8 = F.scales_to_ue8m0(torch.from_numpy(gold["scales_pow2"]).cuda())
    _same(e8.view(torch.uint8).cpu().numpy(), gold["scales_ue8m0"], "UE8M0 bytes")


@pytest.mark.gpu
def test_gemms_match_the_fixtures(gold):
    torch = pytest.importorskip("torch")
    from paddleformers_amd import deep_gemm as DG
    from paddleformers_amd import functional as F

    def f32(bits):
        return O.bf16_bits_to_f32(bits)

    a, sa = G.to_torch_fp8(gold["gemm_a"]), torch.from_numpy(gold["gemm_sa"]).cuda()
    b, sb = G.to_torch_fp8(gold["gemm_b"]), torch.from_numpy(gold["gemm_sb"]).cuda()
    b2, sb2 = G.to_torch_fp8(gold["gemm_b2"]), torch.from_numpy(gold["gemm_sb2"]).cuda()
    out = torch.empty((256, 256), dtype=torch.bfloat16, device="cuda")
    DG.fp8_gemm_nt((a, sa), (b, sb), out)
    assert G.rel_fro(f32(G.from_torch_bf16(out)), f32(gold["gemm_nt_out"])) <= GEMM_FRO
    m_idx = torch.tensor([0] * 128 + [1] * 128, dtype=torch.int32, device="cuda")
    DG.m_grouped_fp8_gemm_nt_contiguous((a, sa), (torch.stack([b.view(torch.uint8), b2.view(torch.uint8)]).view(torch.float8_e4m3fn),
                                                  torch.stack([sb, sb2])), out, m_idx)
    assert G.rel_fro(f32(G.from_torch_bf16(out)), f32(gold["grouped_contig_out"])) <= GEMM_FRO
    om = torch.zeros((2, 128, 256), dtype=torch.bfloat16, device="cuda")
    masked = torch.from_numpy(gold["grouped_masked_m"]).cuda()
    DG.m_grouped_fp8_gemm_nt_masked((a.view(2, 128, 256), sa.view(2, 128, 2)),
                                    (torch.stack([b.view(torch.uint8), b2.view(torch.uint8)]).view(torch.float8_e4m3fn), torch.stack([sb, sb2])),
                                    om, masked, 128)
    got, exp = G.from_torch_bf16(om), gold["grouped_masked_out"]
    for e, v in enumerate(gold["grouped_masked_m"]):
        assert G.rel_fro(f32(got[e, :v]), f32(exp[e, :v])) <= GEMM_FRO
        assert not got[e, v:].any()
    y = F.fp8_gemm_blockwise(G.to_torch_fp8(gold["wgrad_at"]), torch.from_numpy(gold["wgrad_sat"]).cuda(),
                             G.to_torch_fp8(gold["wgrad_bt"]), torch.from_numpy(gold["wgrad_sbt"]).cuda())
    assert G.rel_fro(y.cpu().numpy(), gold["wgrad_out"]) <= 5e-5      # fp32 output: summation order only
