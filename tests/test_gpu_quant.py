"""GPU parity tests of the block quantizers: libpf8 (through the Python mirror of the reference
operator names, i.e. through the C ABI) against the CPU oracle.  Integer/byte outputs and scales
are compared bit for bit."""
import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def F():
    from paddleformers_amd import _lib
    from paddleformers_amd import functional as F8

    _lib.lib()   # fails loudly when libpf8.so has not been built
    return F8


def _same(got, exp, what):
    msg = G.mismatch_report(got, exp, what)
    assert not msg, msg


def _scales_same(got, exp, what):
    # bit-exact: compare the uint32 patterns so that -0/NaN cannot hide
    _same(got.view(np.uint32), exp.view(np.uint32), what)


# ---------------------------------------------------------------------------------------------
# codec and division path
# ---------------------------------------------------------------------------------------------


def _call_debug(name, *tensors_and_n):
    import ctypes as C

    from paddleformers_amd import _lib

    args = []
    for a in tensors_and_n:
        args.append(C.c_void_p(a.data_ptr()) if isinstance(a, torch.Tensor) else a)
    _lib.call(name, *args, C.c_void_p(torch.cuda.current_stream().cuda_stream))


def test_device_sigmoid_of_the_swiglu_backward_matches_the_division(F):
    """1 / (1 + exp(-g)) as the backward kernel forms it (hardware reciprocal, exact residual, one fused correction) against
    the IEEE division of the same denominator, on every finite bf16 g; g / (1 + exp(-g)) from the same reciprocal too."""
    h = np.arange(65536, dtype=np.uint16)
    f = O.bf16_bits_to_f32(h)
    f = f[np.isfinite(f)]
    d = torch.from_numpy(f).cuda()
    sl, sg = torch.empty_like(d), torch.empty_like(d)
    _call_debug("pf8_debug_silu_sigmoid", d, f.size, sl, sg)
    den = (np.float32(1.0) + O.expf_array(-f)).astype(np.float32)
    with np.errstate(all="ignore"):
        want = (np.float32(1.0) / den).astype(np.float32)
    _same(sg.cpu().numpy().view(np.uint32), want.view(np.uint32), "sigmoid over all finite bf16 inputs")
    _same(sl.cpu().numpy().view(np.uint32), O.silu_array(f).view(np.uint32), "silu over all finite bf16 inputs")


def test_hw_encode_matches_oracle_sweep(F):
    """The hardware OCP convert vs the oracle's RNE encoder: every bf16 pattern times a scale
    sweep, the e4m3 grid points, the midpoints between them and their fp32 neighbours."""
    h = np.arange(65536, dtype=np.uint16)
    f = O.bf16_bits_to_f32(h)
    vals = [f]
    for sc in (0.37, 3.3e-3, 17.0, 448.0, 1.0 / 448.0):
        with np.errstate(all="ignore"):
            vals.append((f / np.float32(sc)).astype(np.float32))
    tab = O.e4m3_table()
    grid = np.sort(tab[np.isfinite(tab)]).astype(np.float32)
    mids = ((grid[1:].astype(np.float64) + grid[:-1].astype(np.float64)) / 2).astype(np.float32)
    for base in (grid, mids):
        vals += [base, np.nextafter(base, np.float32(np.inf)), np.nextafter(base, np.float32(-np.inf))]
    v = np.concatenate(vals).astype(np.float32)
    v = v[np.isfinite(v) & (np.abs(v) <= 464.0)]
    # 464 itself is the tie between 448 and the NaN code: the oracle saturates, keep strictly below
    v = v[np.abs(v) < 464.0]
    dv = torch.from_numpy(v).cuda()
    out = torch.empty(v.size, dtype=torch.uint8, device="cuda")
    _call_debug("pf8_debug_encode", dv, v.size, out)
    _same(out.cpu().numpy(), O.e4m3_encode_array(v), "hardware e4m3 encode")


def test_fast_division_path_is_exact(F):
    """e4m3(x / s) through the reciprocal-multiply fast path with its tie guard must equal the
    IEEE-division result, including inputs built to land on and next to rounding boundaries."""
    rng = np.random.default_rng(11)
    n = 1 << 22
    s = np.exp(rng.uniform(np.log(1e-6), np.log(1e3), n)).astype(np.float32)
    x = O.bf16_bits_to_f32(O.f32_to_bf16_bits((rng.uniform(-448, 448, n).astype(np.float32) * s)))
    # adversarial: x = midpoint * s rounded to bf16, s chosen so that the product is exact in bf16
    tab = O.e4m3_table()
    grid = np.sort(tab[np.isfinite(tab) & (tab > 0)])
    mids = ((grid[1:] + grid[:-1]) / 2)
    s2 = (2.0 ** rng.integers(-20, 10, mids.size * 64)).astype(np.float32) * np.float32(1.0)
    m2 = np.tile(mids, 64).astype(np.float32)
    x2 = O.bf16_bits_to_f32(O.f32_to_bf16_bits(m2 * s2))
    # and scales one ulp off a power of two, so the quotient sits a hair off the tie
    s3 = np.nextafter(s2, np.float32(np.inf))
    s4 = np.nextafter(s2, np.float32(0))
    xs = np.concatenate([x, x2, x2, x2, -x2])
    ss = np.concatenate([s, s2, s3, s4, s3])
    keep = np.abs(xs.astype(np.float64) / ss.astype(np.float64)) <= 448.0
    xs, ss = xs[keep], ss[keep]
    dx, ds = torch.from_numpy(xs).cuda(), torch.from_numpy(ss).cuda()
    out = torch.empty(xs.size, dtype=torch.uint8, device="cuda")
    _call_debug("pf8_debug_div_encode", dx, ds, xs.size, out)
    _same(out.cpu().numpy(), O.div_encode_array(xs, ss), "fast division path")


def test_device_silu_matches_oracle(F):
    h = np.arange(65536, dtype=np.uint16)
    f = O.bf16_bits_to_f32(h)
    f = f[np.isfinite(f)]
    d = torch.from_numpy(f).cuda()
    out = torch.empty_like(d)
    _call_debug("pf8_debug_silu", d, f.size, out)
    _same(out.cpu().numpy().view(np.uint32), O.silu_array(f).view(np.uint32), "silu over all finite bf16 inputs")


# ---------------------------------------------------------------------------------------------
# 1x128
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("shape", [(1, 128), (7, 384), (256, 512), (130, 1408), (512, 7168)])
@pytest.mark.parametrize("transpose_scale", [False, True])
@pytest.mark.parametrize("pow2", [False, True])
def test_quant_1x128(F, shape, transpose_scale, pow2):
    bits = G.bf16_normal(shape, seed=shape[0] * 7 + shape[1], outlier_frac=1e-3, outlier_scale=100.0)
    x = G.to_torch_bf16(bits)
    q, s = F.fp8_quant_blockwise(x, quant_method="1x128", input_transpose=False, output_scale_transpose=transpose_scale,
                                 using_pow2_scale=pow2)
    eq, es = O.quant_1x128(bits, scale_layout=int(transpose_scale), pow2=pow2)
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
    assert tuple(s.shape) == es.shape
    _same(G.from_torch_fp8(q), eq, "bytes")
    _scales_same(s.cpu().numpy(), es, "scales")


def test_quant_1x128_config1_full_size(F):
    """BASELINE config 1 activation half: [4096, 7168], N(0,1) + 0.1% outliers x100, seed 0."""
    bits = G.bf16_normal((4096, 7168), seed=0, outlier_frac=1e-3, outlier_scale=100.0)
    x = G.to_torch_bf16(bits)
    q, s = F.fp8_quant_blockwise(x, quant_method="1x128", output_scale_transpose=False)
    eq, es = O.quant_1x128(bits, 0, False)
    _same(G.from_torch_fp8(q), eq, "bytes")
    _scales_same(s.cpu().numpy(), es, "scales")
    # every non-zero tile holds a +-448 byte
    codes = G.from_torch_fp8(q).reshape(4096, 56, 128) & 0x7F
    assert (codes.max(axis=-1) == 0x7E).all()


def test_quant_1x128_edge_tiles(F):
    """All-zero tiles (scale 1, zero bytes), negative zeros, tiny magnitudes whose scale is an
    fp32 subnormal, the largest bf16 values, and a single non-zero element per tile."""
    x = np.zeros((8, 256), dtype=np.float32)
    x[1, :128] = -0.0
    x[2, 5] = 1e-38
    x[2, 6] = -3e-39
    x[3, :] = np.linspace(-1e-40, 1e-40, 256)
    x[4, 0] = 3.38e38
    x[4, 1] = -1.0e38
    x[5, 128 + 17] = -7.0
    x[6, :] = 1.0
    x[7, ::2] = 448.0
    x[7, 1::2] = -0.4375
    bits = O.f32_to_bf16_bits(x)
    bits[1, :128] = 0x8000
    t = G.to_torch_bf16(bits)
    for pow2 in (False, True):
        q, s = F.fp8_quant_blockwise(t, quant_method="1x128", using_pow2_scale=pow2)
        eq, es = O.quant_1x128(bits, 0, pow2)
        _same(G.from_torch_fp8(q), eq, f"bytes pow2={pow2}")
        _scales_same(s.cpu().numpy(), es, f"scales pow2={pow2}")
    assert s[0, 0].item() == 1.0 and (G.from_torch_fp8(q)[0] == 0).all()
    assert (G.from_torch_fp8(q)[1, :128] == 0x80).all()


def test_quant_1x128_rejects_bad_shapes(F):
    x = torch.zeros((4, 200), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        F.fp8_quant_blockwise(x, quant_method="1x128")
    with pytest.raises(RuntimeError):
        F.fp8_quant_blockwise(torch.zeros((4, 128), dtype=torch.bfloat16), quant_method="1x128")
    q, s = F.fp8_quant_blockwise(torch.zeros((0, 256), dtype=torch.bfloat16, device="cuda"), quant_method="1x128")
    assert tuple(q.shape) == (0, 256) and tuple(s.shape) == (0, 2)


# ---------------------------------------------------------------------------------------------
# 128x128 and stacked weights
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("shape", [(128, 128), (256, 384), (1408, 512)])
@pytest.mark.parametrize("pow2", [False, True])
def test_quant_128x128_all_return_forms(F, shape, pow2):
    bits = G.bf16_normal(shape, seed=sum(shape), std=0.02, outlier_frac=5e-4, outlier_scale=50.0)
    w = G.to_torch_bf16(bits)
    eq, es, eqt, est = O.quant_128x128(bits, want=(True, True), pow2=pow2)
    q, s = F.fp8_quant_blockwise(w, quant_method="128x128", using_pow2_scale=pow2)
    _same(G.from_torch_fp8(q), eq, "q")
    _scales_same(s.cpu().numpy(), es, "s")
    q, s, qt, st = F.fp8_quant_blockwise(w, quant_method="128x128", input_transpose=True, using_pow2_scale=pow2)
    _same(G.from_torch_fp8(q), eq, "q (4-out)")
    _same(G.from_torch_fp8(qt), eqt, "q_t (4-out)")
    _scales_same(s.cpu().numpy(), es, "s (4-out)")
    _scales_same(st.cpu().numpy(), est, "s_t (4-out)")
    qt, st = F.fp8_quant_blockwise(w, quant_method="128x128", input_transpose=True, return_transpose_only=True,
                                   using_pow2_scale=pow2)
    _same(G.from_torch_fp8(qt), eqt, "q_t (transpose only)")
    _scales_same(st.cpu().numpy(), est, "s_t (transpose only)")
    # the identity the reference relies on (fp8_utils.py:110,123)
    _same(G.from_torch_fp8(qt), eq.T, "q_t == q^T")


def test_quant_128x128_config1_weight(F):
    bits = G.bf16_normal((7168, 2048), seed=0, outlier_frac=1e-3, outlier_scale=100.0)
    w = G.to_torch_bf16(bits)
    q, s = F.fp8_quant_blockwise(w, quant_method="128x128")
    eq, es, _, _ = O.quant_128x128(bits)
    _same(G.from_torch_fp8(q), eq, "bytes")
    _scales_same(s.cpu().numpy(), es, "scales")
    assert tuple(s.shape) == (56, 16)


@pytest.mark.parametrize("transpose", [False, True])
def test_fused_stack_transpose_quant(F, transpose):
    E, R, C = 5, 256, 384
    ws = [G.bf16_normal((R, C), seed=100 + e, std=0.02, outlier_frac=1e-3, outlier_scale=50.0) for e in range(E)]
    q, s = F.fused_stack_transpose_quant([G.to_torch_bf16(w) for w in ws], transpose=transpose)
    eq, es = O.stack_transpose_quant(ws, transpose=transpose)
    assert tuple(q.shape) == eq.shape and tuple(s.shape) == es.shape
    _same(G.from_torch_fp8(q), eq, "stacked bytes")
    _scales_same(s.cpu().numpy(), es, "stacked scales")


def test_fused_stack_quant_both_equals_two_calls(F):
    """One read, both orientations: bytes and scales of the oracle's two separate quantizations."""
    E, R, C = 5, 256, 384
    ws = [G.bf16_normal((R, C), seed=300 + e, std=0.02, outlier_frac=1e-3, outlier_scale=50.0) for e in range(E)]
    q, s, qt, st = F.fused_stack_quant_both([G.to_torch_bf16(w) for w in ws])
    eq, es = O.stack_transpose_quant(ws, transpose=False)
    eqt, est = O.stack_transpose_quant(ws, transpose=True)
    _same(G.from_torch_fp8(q), eq, "stacked bytes")
    _scales_same(s.cpu().numpy(), es, "stacked scales")
    _same(G.from_torch_fp8(qt), eqt, "stacked transposed bytes")
    _scales_same(st.cpu().numpy(), est, "stacked transposed scales")


@pytest.mark.parametrize("want", [(True, True), (True, False), (False, True)])
def test_fused_stack_quant_both_writes_fragment_major_copies(F, want):
    """The copies made in the quantizer's pass are the bytes the re-ordering pass makes of its plain outputs."""
    from paddleformers_amd import deep_gemm as dg

    E, R, C = 3, 256, 384
    ws = [G.to_torch_bf16(G.bf16_normal((R, C), seed=320 + e, std=0.02, outlier_frac=1e-3, outlier_scale=50.0)) for e in range(E)]
    q0, s0, qt0, st0 = F.fused_stack_quant_both(ws)
    q, s, qt, st, q_fm, qt_fm = F.fused_stack_quant_both(ws, fragment_major=want)
    for a, b in ((q, q0), (qt, qt0)):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    assert torch.equal(s, s0) and torch.equal(st, st0)
    assert (q_fm is not None, qt_fm is not None) == want
    if q_fm is not None:
        assert torch.equal(q_fm.view(torch.uint8).view(E, R, C), dg.to_fragment_major(q.view(E, R, C)).data.view(torch.uint8))
    if qt_fm is not None:
        assert torch.equal(qt_fm.view(torch.uint8).view(E, C, R), dg.to_fragment_major(qt.view(E, C, R)).data.view(torch.uint8))
    assert F.fused_stack_quant_both(ws, fragment_major=(False, False))[4:] == (None, None)


def test_fp8_quant_weight_caches_what_fused_stack_quant_reads():
    """The per-step requantization caller (modeling.py:506-567): batch mode attaches both
    orientations to expert 0's weights, and fused_stack_quant then serves them from the cache."""
    from paddleformers_amd import fp8_utils as U
    from paddleformers_amd import functional as F8

    E, H, I = 3, 256, 128
    w1 = [G.to_torch_bf16(G.bf16_normal((H, 2 * I), seed=400 + e, std=0.02)) for e in range(E)]
    w2 = [G.to_torch_bf16(G.bf16_normal((I, H), seed=500 + e, std=0.02)) for e in range(E)]
    ref = F8.fused_stack_transpose_quant(w1, transpose=True)
    ref2 = F8.fused_stack_transpose_quant(w2, transpose=False)
    U.fp8_quant_weight(w1, w2, batch_mode=True, quant_transpose=None)
    q, s = U.fused_stack_quant(w1, transpose=True)
    assert q is w1[0].fp8_weight_stacked_transpose
    assert torch.equal(q.view(torch.uint8), ref[0].view(torch.uint8)) and torch.equal(s, ref[1])
    q, s = U.fused_stack_quant(w2, transpose=False)
    assert q is w2[0].fp8_weight_stacked
    assert torch.equal(q.view(torch.uint8), ref2[0].view(torch.uint8)) and torch.equal(s, ref2[1])
    with pytest.raises(ValueError):
        U.fp8_quant_weight([G.to_torch_bf16(G.bf16_normal((128, 128), seed=1))], [G.to_torch_bf16(G.bf16_normal((128, 128), seed=2))],
                           quant_transpose="both")


@pytest.mark.parametrize("quant_transpose", [None, False, True])
def test_fp8_quant_weight_all_layers_equals_the_per_layer_calls(quant_transpose):
    """Every MoE layer's batch-mode cache from one launch per weight shape: same tensors as
    fp8_quant_weight(batch_mode=True) layer by layer, and lists that are already cached are skipped."""
    from paddleformers_amd import fp8_utils as U

    E, H, I, L = 2, 256, 128, 3

    def make(seed):
        return ([G.to_torch_bf16(G.bf16_normal((H, 2 * I), seed=seed + e, std=0.02)) for e in range(E)],
                [G.to_torch_bf16(G.bf16_normal((I, H), seed=seed + 50 + e, std=0.02)) for e in range(E)])

    layers, refs = [make(600 + 100 * i) for i in range(L)], [make(600 + 100 * i) for i in range(L)]
    for w1, w2 in refs:
        U.fp8_quant_weight(w1, w2, batch_mode=True, quant_transpose=quant_transpose)
    sentinel = object()
    layers[1][1][0].fp8_weight_stacked = sentinel            # this list already has a cache
    U.fp8_quant_weight_all_layers(layers, quant_transpose=quant_transpose)
    assert layers[1][1][0].fp8_weight_stacked is sentinel and not hasattr(layers[1][1][0], "fp8_scale_stacked")
    names = {None: ["fp8_weight_stacked", "fp8_scale_stacked", "fp8_weight_stacked_transpose", "fp8_scale_stacked_transpose"],
             False: ["fp8_weight_stacked", "fp8_scale_stacked"], True: ["fp8_weight_stacked_transpose", "fp8_scale_stacked_transpose"]}[quant_transpose]
    for li in range(L):
        for k in (0, 1):
            if (li, k) == (1, 1):
                continue
            got, ref = layers[li][k][0], refs[li][k][0]
            for n in names:
                a, b = getattr(got, n), getattr(ref, n)
                assert a.shape == b.shape and torch.equal(a.view(torch.uint8) if a.dtype != torch.float32 else a,
                                                          b.view(torch.uint8) if b.dtype != torch.float32 else b), (li, k, n)
            assert got.fp8_scale_is_pow2 is False
            assert not hasattr(layers[li][k][1], "fp8_weight_stacked")      # batch mode: only the first weight carries the cache


# ---------------------------------------------------------------------------------------------
# fused quant + transpose
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("shape", [(128, 128), (384, 256), (512, 1408)])
@pytest.mark.parametrize("transpose_scale", [False, True])
def test_quant_transpose_equals_two_quantizations(F, shape, transpose_scale):
    bits = G.bf16_normal(shape, seed=shape[0] + 3 * shape[1], outlier_frac=1e-3, outlier_scale=100.0)
    x = G.to_torch_bf16(bits)
    q, s, qt, st = F.fp8_quant_blockwise(x, quant_method="1x128", input_transpose=True, output_scale_transpose=transpose_scale)
    lay = int(transpose_scale)
    eq, es = O.quant_1x128(bits, lay)
    eqt, est = O.quant_1x128(np.ascontiguousarray(bits.T), lay)
    _same(G.from_torch_fp8(q), eq, "row-scaled bytes")
    _scales_same(s.cpu().numpy(), es, "row scales")
    _same(G.from_torch_fp8(qt), eqt, "column-scaled transposed bytes")
    _scales_same(st.cpu().numpy(), est, "column scales")
    qt2, st2 = F.fp8_quant_blockwise(x, quant_method="1x128", input_transpose=True, output_scale_transpose=transpose_scale,
                                     return_transpose_only=True)
    _same(G.from_torch_fp8(qt2), eqt, "transpose-only bytes")
    _scales_same(st2.cpu().numpy(), est, "transpose-only scales")


def test_quant_transpose_config4_full_size_property(F):
    """BASELINE config 4 at full size [16384, 7168]: the fused kernel must equal the 1x128
    quantizer applied to x and to x^T (a size-independent property checked on the GPU), and a
    2048-row slab is checked against the CPU oracle."""
    bits = G.bf16_normal((16384, 7168), seed=4, outlier_frac=1e-3, outlier_scale=100.0)
    x = G.to_torch_bf16(bits)
    q, s, qt, st = F.fp8_quant_blockwise(x, quant_method="1x128", input_transpose=True, output_scale_transpose=True)
    q1, s1 = F.fp8_quant_blockwise(x, quant_method="1x128", output_scale_transpose=True)
    q2, s2 = F.fp8_quant_blockwise(x.t().contiguous(), quant_method="1x128", output_scale_transpose=True)
    assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8))
    assert torch.equal(s.view(torch.int32), s1.view(torch.int32))
    assert torch.equal(qt.view(torch.uint8), q2.view(torch.uint8))
    assert torch.equal(st.view(torch.int32), s2.view(torch.int32))
    eq, es = O.quant_1x128(bits[:2048], 0)
    _same(G.from_torch_fp8(q[:2048]), eq, "slab bytes vs oracle")
    _scales_same(s.t()[:2048].contiguous().cpu().numpy(), es, "slab scales vs oracle")
    # the column-scaled copy straight against the oracle as well: 1024 columns of x = 1024 rows of the transposed output
    eqt, est = O.quant_1x128(np.ascontiguousarray(bits[:, 1024:2048].T), 1)
    _same(G.from_torch_fp8(qt[1024:2048]), eqt, "column-scaled slab bytes vs oracle")
    _scales_same(st[:, 1024:2048].contiguous().cpu().numpy(), est, "column-scaled slab scales vs oracle")


def test_padding_and_quant_input_unaligned_rows(F):
    """fp8_utils.py:155-174: rows not a multiple of 512 -> row copy from the unpadded tensor,
    transposed copy from the zero-padded one."""
    from paddleformers_amd.fp8_utils import FP8LinearFunctionBase as B

    bits = G.bf16_normal((300, 256), seed=9)
    x = G.to_torch_bf16(bits)
    q, s, qt, st = B.padding_and_quant_input(x)
    assert tuple(q.shape) == (300, 256) and tuple(qt.shape) == (256, 512) and tuple(st.shape) == (4, 256)
    padded = np.zeros((512, 256), np.uint16)
    padded[:300] = bits
    eq, es = O.quant_1x128(bits, 1)
    eqt, est = O.quant_1x128(np.ascontiguousarray(padded.T), 1)
    _same(G.from_torch_fp8(q), eq, "row bytes")
    _same(G.from_torch_fp8(qt), eqt, "padded transposed bytes")
    _scales_same(st.cpu().numpy(), est, "padded transposed scales")
    for n, exp in ((300, 512), (512, 512), (640, 1024), (1, 512), (513, 1024), (900, 1024)):
        assert B.padding(torch.zeros((n, 8), device="cuda"), 0).shape[0] == exp


# ---------------------------------------------------------------------------------------------
# fused SwiGLU + requant
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("M,I", [(5, 128), (130, 256), (256, 1408), (512, 2048)])
@pytest.mark.parametrize("with_probs", [False, True])
@pytest.mark.parametrize("pow2", [False, True])
def test_fused_weighted_swiglu_act_quant(F, M, I, with_probs, pow2):
    bits = G.bf16_normal((M, 2 * I), seed=M + I, std=2.0, outlier_frac=1e-3, outlier_scale=20.0)
    rng = np.random.default_rng(M)
    probs = rng.random(M, dtype=np.float32) if with_probs else None
    o1 = G.to_torch_bf16(bits)
    tp = torch.from_numpy(probs).cuda() if with_probs else None
    q, s, o2 = F.fused_weighted_swiglu_act_quant(o1, tp, using_pow2_scaling=pow2, return_o2=True)
    eq, es, eo2 = O.swiglu_weighted_quant(bits, probs, 0, pow2, return_o2=True)
    _same(G.from_torch_bf16(o2), eo2, "bf16 activations")
    _same(G.from_torch_fp8(q), eq, "bytes")
    _scales_same(s.cpu().numpy(), es, "scales")


def test_swiglu_probs_column_vector_and_zero_rows(F):
    o1 = G.to_torch_bf16(G.bf16_normal((128, 256), seed=1))
    p = torch.rand(128, 1, device="cuda")
    q1, s1 = F.fused_weighted_swiglu_act_quant(o1, p, using_pow2_scaling=True)
    q2, s2 = F.fused_weighted_swiglu_act_quant(o1, p.squeeze(-1), using_pow2_scaling=True)
    assert torch.equal(q1.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s1, s2)
    # pow2 scales are powers of two
    m, _ = np.frexp(s1.cpu().numpy())
    assert (m == 0.5).all()
    q, s = F.fused_weighted_swiglu_act_quant(torch.zeros((0, 256), dtype=torch.bfloat16, device="cuda"), None)
    assert tuple(q.shape) == (0, 128)


# ---------------------------------------------------------------------------------------------
# transpose + split + quant
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("rows", [[128], [256, 0, 128], [0, 0, 384, 128, 0], [128] * 7])
@pytest.mark.parametrize("pow2", [False, True])
def test_fused_transpose_split_quant_bf16(F, rows, pow2):
    K = 384
    M = sum(rows)
    bits = G.bf16_normal((M, K), seed=M + len(rows), outlier_frac=1e-3, outlier_scale=100.0)
    qs, ss = F.fused_transpose_split_quant(G.to_torch_bf16(bits), None, rows, pow2)
    eqs, ess = O.transpose_split_quant(bits, None, rows, pow2)
    assert len(qs) == len(rows)
    for e, r in enumerate(rows):
        assert tuple(qs[e].shape) == (K, r) and tuple(ss[e].shape) == (r // 128, K)
        if r:
            _same(G.from_torch_fp8(qs[e]), eqs[e], f"expert {e} bytes")
            _scales_same(ss[e].cpu().numpy(), ess[e], f"expert {e} scales")


@pytest.mark.parametrize("scale_transposed", [False, True])
def test_fused_transpose_split_quant_fp8_input(F, scale_transposed):
    rows = [256, 0, 128, 384]
    K = 512
    M = sum(rows)
    bits = G.bf16_normal((M, K), seed=77, outlier_frac=1e-3, outlier_scale=100.0)
    xq, xs = O.quant_1x128(bits, 0)
    tq = G.to_torch_fp8(xq)
    if scale_transposed:
        ts = torch.from_numpy(np.ascontiguousarray(xs.T)).cuda().t()   # [M, K/128] view of [K/128, M]
    else:
        ts = torch.from_numpy(xs).cuda()
    qs, ss = F.fused_transpose_split_quant(tq, ts, rows, True)
    eqs, ess = O.transpose_split_quant(xq, xs, rows, True)
    for e, r in enumerate(rows):
        if r:
            _same(G.from_torch_fp8(qs[e]), eqs[e], f"expert {e} bytes")
            _scales_same(ss[e].cpu().numpy(), ess[e], f"expert {e} scales")


@pytest.mark.parametrize("rows", [[128], [256, 0, 128], [0, 0, 384, 128, 0]])
@pytest.mark.parametrize("pow2_rows", [False, True])
def test_quant_and_transpose_split_equals_the_two_separate_quantizers(F, rows, pow2_rows):
    # one read, both quantizations of the MoE backward: row-wise 1x128 (scales [K/128, M]) and the
    # per-expert transposed copy with power-of-two scales
    K = 384
    M = sum(rows)
    bits = G.bf16_normal((M, K), seed=3 * M + len(rows), outlier_frac=1e-3, outlier_scale=100.0)
    q, s, qs, ss = F.quant_and_transpose_split(G.to_torch_bf16(bits), rows, pow2_rows, True)
    eq, es = O.quant_1x128(bits, 1, pow2=pow2_rows)
    _same(G.from_torch_fp8(q), eq, "row-wise bytes")
    _scales_same(s.cpu().numpy(), es, "row-wise scales")
    eqs, ess = O.transpose_split_quant(bits, None, rows, True)
    for e, r in enumerate(rows):
        assert tuple(qs[e].shape) == (K, r) and tuple(ss[e].shape) == (r // 128, K)
        if r:
            _same(G.from_torch_fp8(qs[e]), eqs[e], f"expert {e} bytes")
            _scales_same(ss[e].cpu().numpy(), ess[e], f"expert {e} scales")
    # and against the library's own separate entry points
    q1, s1 = F.fp8_quant_blockwise(G.to_torch_bf16(bits), output_scale_transpose=True, quant_method="1x128", input_transpose=False,
                                   using_pow2_scale=pow2_rows)
    assert torch.equal(q1.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s1, s)


def test_quant_and_transpose_split_rejects_bad_input(F):
    x = torch.zeros((256, 256), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        F.quant_and_transpose_split(x, [128, 64, 64])
    with pytest.raises(ValueError):
        F.quant_and_transpose_split(x, [128])
    with pytest.raises(ValueError):
        F.quant_and_transpose_split(x.float(), [256])
    q, s, qs, ss = F.quant_and_transpose_split(torch.zeros((0, 256), dtype=torch.bfloat16, device="cuda"), [0, 0])
    assert tuple(q.shape) == (0, 256) and len(qs) == 2


# ---------------------------------------------------------------------------------------------
# dequantizers and SwiGLU backward
# ---------------------------------------------------------------------------------------------


def test_fused_act_dequant(F):
    bits = G.bf16_normal((200, 640), seed=5, outlier_frac=1e-3, outlier_scale=100.0)
    q, s = O.quant_1x128(bits, 0)
    out = F.fused_act_dequant(G.to_torch_fp8(q), torch.from_numpy(s).cuda())
    _same(G.from_torch_bf16(out), O.act_dequant(q, s, 0), "dequant (row-major scales)")
    st = torch.from_numpy(np.ascontiguousarray(s.T)).cuda().t()
    out = F.fused_act_dequant(G.to_torch_fp8(q), st)
    _same(G.from_torch_bf16(out), O.act_dequant(q, s, 0), "dequant (transposed scales)")
    # all 256 codes, including the NaN code and the subnormals
    codes = np.tile(np.arange(256, dtype=np.uint8), 128).reshape(256, 128)
    sc = np.linspace(0.5, 3.0, 256, dtype=np.float32).reshape(256, 1)
    got = G.from_torch_bf16(F.fused_act_dequant(G.to_torch_fp8(codes), torch.from_numpy(sc).cuda()))
    exp = O.act_dequant(codes, sc, 0)
    nan = (codes & 0x7F) == 0x7F
    _same(got[~nan], exp[~nan], "all codes")
    assert np.isnan(O.bf16_bits_to_f32(got[nan])).all()


def test_weight_dequant_with_ragged_edges(F):
    """The reference's block-dequant KATs (trailing partial block cropped) plus a random case."""
    rng = np.random.default_rng(3)
    for R, C in ((256, 384), (3, 3), (130, 257)):
        q = rng.integers(0, 0x7F, (R, C), dtype=np.uint8) | (rng.integers(0, 2, (R, C), dtype=np.uint8) << 7)
        q[(q & 0x7F) == 0x7F] = 0x38
        s = rng.random(((R + 127) // 128, (C + 127) // 128), dtype=np.float32) + 0.5
        out = F.weight_dequant(torch.from_numpy(q).cuda(), torch.from_numpy(s).cuda())
        _same(G.from_torch_bf16(out), O.weight_dequant(q, s), f"weight dequant {R}x{C}")


def test_fused_swiglu_weighted_bwd(F):
    M, I = 130, 256
    o1 = G.bf16_normal((M, 2 * I), seed=21, std=1.5)
    do2 = G.bf16_normal((M, I), seed=22, std=1e-3)
    probs = np.random.default_rng(23).random(M, dtype=np.float32)
    do1, pg, o2s = F.fused_swiglu_weighted_bwd(G.to_torch_bf16(o1), G.to_torch_bf16(do2), torch.from_numpy(probs).cuda())
    edo1, epg, eo2s = O.swiglu_weighted_bwd(o1, do2, probs)
    _same(G.from_torch_bf16(o2s), eo2s, "o2_s")
    _same(G.from_torch_bf16(do1), edo1, "do1")
    # probs_grad is a 256-term fp32 sum whose order differs from the oracle's float64 sum:
    # tolerance 1e-5 of the row's absolute-term sum
    terms = np.abs(O.bf16_bits_to_f32(do2).astype(np.float64)).sum(axis=1) * 8.0
    assert np.all(np.abs(pg.cpu().numpy().astype(np.float64) - epg) <= 1e-5 * terms + 1e-30)


# ---------------------------------------------------------------------------------------------
# UE8M0 exponent bytes written by the quantizers themselves
# ---------------------------------------------------------------------------------------------


def _e8_of(scale_f32):
    """Power-of-two fp32 scales -> UE8M0 bytes (the biased exponent field)."""
    bits = np.ascontiguousarray(scale_f32).view(np.uint32)
    assert (bits & 0x807FFFFF == 0).all(), "not powers of two"
    return (bits >> 23).astype(np.uint8)


@pytest.mark.parametrize("M,K", [(4, 128), (136, 1408), (515, 512)])
@pytest.mark.parametrize("transpose", [False, True])
def test_quant_1x128_writes_ue8m0_bytes(F, M, K, transpose):
    bits = G.bf16_normal((M, K), seed=M + K, outlier_frac=1e-3, outlier_scale=300.0)
    bits[1, :128] = 0                                   # an all-zero tile: scale 1 = byte 127
    bits[2, :128] = G.bf16_normal((128,), seed=3, std=1e-30)          # tiny values: the scale rule's division path
    eq, es = O.quant_1x128(bits, 0, True)
    x = G.to_torch_bf16(bits)
    q, s = F.fp8_quant_blockwise(x, quant_method="1x128", using_pow2_scale=True, output_scale_transpose=transpose, ue8m0_scale=True)
    assert s.dtype == torch.uint8 and tuple(s.shape) == ((K // 128, M) if transpose else (M, K // 128))
    got = s.cpu().numpy()
    _same(G.from_torch_fp8(q), eq, "bytes")
    _same(got.T if transpose else got, _e8_of(es), "exponent bytes")
    assert got[(0, 1) if transpose else (1, 0)] == 127
    # the conversion pass is the identity on bytes
    assert F.scales_to_ue8m0(s) is s
    with pytest.raises(ValueError):
        F.fp8_quant_blockwise(x, quant_method="1x128", using_pow2_scale=False, ue8m0_scale=True)


def test_swiglu_quant_writes_ue8m0_bytes(F):
    M, I = 260, 512
    o1 = G.bf16_normal((M, 2 * I), seed=5, std=2.0)
    probs = np.random.default_rng(6).random(M).astype(np.float32)
    eq, es = O.swiglu_weighted_quant(o1, probs, pow2=True)
    q, s = F.fused_weighted_swiglu_act_quant(G.to_torch_bf16(o1), torch.from_numpy(probs).cuda(), using_pow2_scaling=True, ue8m0_scale=True)
    assert s.dtype == torch.uint8 and tuple(s.shape) == (M, I // 128) and s.stride() == (1, M)
    _same(G.from_torch_fp8(q), eq, "bytes")
    _same(s.cpu().numpy(), _e8_of(es), "exponent bytes")
    with pytest.raises(ValueError):
        F.fused_weighted_swiglu_act_quant(G.to_torch_bf16(o1), None, using_pow2_scaling=False, ue8m0_scale=True)


def test_quant_and_transpose_split_writes_ue8m0_row_scales_and_reads_them_back(F):
    rows, K = [128, 0, 256], 640
    bits = G.bf16_normal((sum(rows), K), seed=8, outlier_frac=1e-3, outlier_scale=100.0)
    x = G.to_torch_bf16(bits)
    q0, s0, qt0, st0 = F.quant_and_transpose_split(x, rows, True, True)
    q1, s1, qt1, st1 = F.quant_and_transpose_split(x, rows, True, True, ue8m0_scale=True)
    assert s1.dtype == torch.uint8 and s1.shape == s0.shape
    assert torch.equal(q0.view(torch.uint8), q1.view(torch.uint8))
    _same(s1.cpu().numpy(), _e8_of(s0.cpu().numpy()), "row-scale exponent bytes")
    for a, b in zip(qt0 + st0, qt1 + st1):
        assert torch.equal(a.view(torch.uint8) if a.dtype != torch.float32 else a, b.view(torch.uint8) if b.dtype != torch.float32 else b)
    # the transposed quantizer of an e4m3 input takes its scales as bytes (what the node caches in that mode)
    qa, sa = F.fused_transpose_split_quant(q0, s0.T, rows, True)
    qb, sb = F.fused_transpose_split_quant(q1, s1.T, rows, True)
    for a, b in zip(qa + sa, qb + sb):
        assert torch.equal(a.view(torch.uint8) if a.dtype != torch.float32 else a, b.view(torch.uint8) if b.dtype != torch.float32 else b)
    with pytest.raises(ValueError):
        F.quant_and_transpose_split(x, rows, False, True, ue8m0_scale=True)
