"""GPU parity tests of the FP8 GEMMs whose scales are UE8M0 exponent bytes (power-of-two scales
applied inside gfx950's block-scaled MFMA), through the deep_gemm-named mirror and the C ABI.

The oracle is the same one the fp32-scale GEMMs are checked against, fed the decoded scales
(2^(byte-127), a table pinned by the reference's known-answer vectors); tolerances as in
tests/test_gpu_gemm.py: relative Frobenius <= 1e-3 against bf16(dequant(a) @ dequant(b)^T) and the
per-element bound.  The bound against the block-accumulating oracle is 8e-4 instead of 6e-4: here
the matrix pipe accumulates across K blocks itself, in its own order, instead of the per-block FMA
that oracle restates, so a few more bf16 outputs round the other way (one flip is 2^-8 relative;
8e-4 allows 4% of the elements to flip and is still far below any scale or indexing mistake).
For the same reason the per-element slack is 8e-5 of sum|a||b| (6e-5 for the fp32-scale kernels;
measured worst case here 4.4e-5 with the running sum kept inside the matrix pipe)."""
import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

REL_FRO = 1e-3
BLOCK_FRO = 8e-4
ELEM_ABS = 8e-5


@pytest.fixture(scope="module")
def dg():
    from paddleformers_amd import _lib, deep_gemm

    _lib.lib()
    return deep_gemm


def _bf(bits):
    return O.bf16_bits_to_f32(bits)


def _pow2_case(M, N, K, seed, std_w=0.02):
    xa = G.bf16_normal((M, K), seed=seed, outlier_frac=1e-3, outlier_scale=30.0)
    wb = G.bf16_normal((N, K), seed=seed + 1, std=std_w, outlier_frac=5e-4, outlier_scale=50.0)
    a, sa = O.quant_1x128(xa, 0, pow2=True)
    b, sb, _, _ = O.quant_128x128(wb, pow2=True)
    return a, sa, b, sb


def _elementwise_ok(got_f32, a, sa, b, sb, what):
    af = O.e4m3_decode_np(a).astype(np.float64) * np.repeat(sa.astype(np.float64), 128, axis=1)
    bf = O.e4m3_decode_np(b).astype(np.float64) * np.repeat(np.repeat(sb.astype(np.float64), 128, axis=0), 128, axis=1)[: b.shape[0]]
    exact = af @ bf.T
    tol = ELEM_ABS * (np.abs(af) @ np.abs(bf).T) + 2.0 ** -8 * np.abs(exact) + 1e-30
    err = np.abs(got_f32.astype(np.float64) - exact)
    bad = np.argwhere(err > tol)
    worst = float(np.max((err - 2.0 ** -8 * np.abs(exact)) / (np.abs(af) @ np.abs(bf).T + 1e-30)))
    assert bad.size == 0, f"{what}: {len(bad)} elements outside tolerance (worst excess {worst:.2e} of sum|a||b|), first at {tuple(bad[0])}"


def _check(got_bits, a, sa, b, sb, what):
    ref = O.gemm_nt(a, sa, b, sb, dequant_ref=True)
    blk = O.gemm_nt(a, sa, b, sb)
    assert G.rel_fro(_bf(got_bits), _bf(ref)) <= REL_FRO, what
    assert G.rel_fro(_bf(got_bits), _bf(blk)) <= BLOCK_FRO, what
    _elementwise_ok(_bf(got_bits), a, sa, b, sb, what)


def _e8(s):
    return torch.from_numpy(O.scales_to_ue8m0(s)).cuda()


def test_scales_to_ue8m0_matches_oracle_and_rejects_other_scales():
    from paddleformers_amd import functional as F

    xa = G.bf16_normal((384, 1024), seed=11, outlier_frac=1e-3, outlier_scale=100.0)
    _, s = O.quant_1x128(xa, 1, pow2=True)
    got = F.scales_to_ue8m0(torch.from_numpy(s).cuda())
    assert got.dtype == torch.uint8 and tuple(got.shape) == s.shape
    assert np.array_equal(got.cpu().numpy(), O.scales_to_ue8m0(s))
    # the M-contiguous view keeps its layout
    got_t = F.scales_to_ue8m0(torch.from_numpy(s).cuda().t())
    assert got_t.stride() == (1, s.shape[1]) and np.array_equal(got_t.cpu().numpy(), O.scales_to_ue8m0(s).T)
    _, s_np2 = O.quant_1x128(xa, 0, pow2=False)
    with pytest.raises(ValueError):
        F.scales_to_ue8m0(torch.from_numpy(s_np2).cuda())
    with pytest.raises(ValueError):
        F.scales_to_ue8m0(torch.tensor([1.0, 0.0, -2.0], device="cuda"))


# 384 and 640 rows end in a half tile; 128 is a lone half tile; 384, 640 and 1408 columns end in a half tile
@pytest.mark.parametrize("M,N,K", [(256, 256, 384), (512, 768, 1024), (384, 512, 512), (128, 256, 640), (640, 1024, 896),
                                   (256, 384, 512), (384, 640, 640), (512, 1408, 384)])
@pytest.mark.parametrize("kmajor", [False, True])
def test_gemm_nt_ue8m0_vs_oracle(dg, M, N, K, kmajor):
    a, sa, b, sb = _pow2_case(M, N, K, seed=M + N + K)
    tsa = _e8(np.ascontiguousarray(sa.T)).t() if kmajor else _e8(sa)     # logical [M, K/128] either way
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    dg.fp8_gemm_nt((G.to_torch_fp8(a), tsa), (G.to_torch_fp8(b), _e8(sb)), out)
    _check(G.from_torch_bf16(out), a, sa, b, sb, f"ue8m0 gemm {M}x{N}x{K}")


@pytest.mark.parametrize("N", [512, 640])
def test_gemm_nt_ue8m0_scales_are_applied_per_row_and_block(dg, N):
    """Ones times ones with a distinct exponent for every (row, K block) and (column block, K block):
    the result is sum_kb 128 * 2^(ea[m,kb] + eb[n/128,kb]) exactly -- catches a transposed, mis-selected
    (op_sel) or mis-indexed scale byte and a wrong row permutation inside a fragment."""
    M, K = 512, 512
    rng = np.random.default_rng(5)
    one = O.e4m3_encode_array(np.ones(1, np.float32))[0]
    a = np.full((M, K), one, np.uint8)
    b = np.full((N, K), one, np.uint8)
    ea = rng.integers(124, 132, (M, K // 128)).astype(np.uint8)
    eb = rng.integers(125, 131, (N // 128, K // 128)).astype(np.uint8)
    out = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    dg.fp8_gemm_nt((G.to_torch_fp8(a), torch.from_numpy(ea).cuda()), (G.to_torch_fp8(b), torch.from_numpy(eb).cuda()), out)
    sa, sb = O.decode_scales(ea, "ue8m0").astype(np.float64), O.decode_scales(eb, "ue8m0").astype(np.float64)
    exp = 128.0 * (sa @ np.repeat(sb, 128, axis=0).T)
    assert np.array_equal(G.from_torch_bf16(out), O.f32_to_bf16_bits(exp.astype(np.float32)))


def test_gemm_nt_ue8m0_exact_integer_case_with_row_stride(dg):
    """Small integers and unit scales: an exact integer matmul, written into a wider output."""
    rng = np.random.default_rng(0)
    M, N, K = 256, 512, 384
    ai, bi = rng.integers(-3, 4, (M, K)), rng.integers(-2, 3, (N, K))
    a = O.e4m3_encode_array(ai.astype(np.float32))
    b = O.e4m3_encode_array(bi.astype(np.float32))
    ea = np.full((M, K // 128), 127, np.uint8)
    eb = np.full((N // 128, K // 128), 127, np.uint8)
    wide = torch.full((M, N + 64), 5.0, dtype=torch.bfloat16, device="cuda")
    dg.fp8_gemm_nt((G.to_torch_fp8(a), torch.from_numpy(ea).cuda()), (G.to_torch_fp8(b), torch.from_numpy(eb).cuda()), wide[:, :N])
    assert np.array_equal(G.from_torch_bf16(wide[:, :N].contiguous()), O.f32_to_bf16_bits((ai @ bi.T).astype(np.float32)))
    assert (wide[:, N:] == 5.0).all()


@pytest.mark.parametrize("M,N,K", [(200, 384, 256), (256, 128, 512), (256, 256, 256)])
def test_gemm_nt_ue8m0_other_shapes_take_the_decoded_scale_kernel(dg, M, N, K):
    """Shapes outside the block-scaled kernel's tiling give the same result through the fp32-scale kernel."""
    a, sa, b, sb = _pow2_case(M, N, K, seed=7)
    out = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    dg.fp8_gemm_nt((G.to_torch_fp8(a), _e8(sa)), (G.to_torch_fp8(b), _e8(sb)), out)
    ref = torch.empty_like(out)
    dg.fp8_gemm_nt((G.to_torch_fp8(a), torch.from_numpy(sa).cuda()), (G.to_torch_fp8(b), torch.from_numpy(sb).cuda()), ref)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def test_gemm_nt_ue8m0_rejects_mixed_scale_kinds(dg):
    a, sa, b, sb = _pow2_case(256, 256, 384, seed=9)
    out = torch.empty((256, 256), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        dg.fp8_gemm_nt((G.to_torch_fp8(a), _e8(sa)), (G.to_torch_fp8(b), torch.from_numpy(sb).cuda()), out)


def _grouped_pow2_case(E, N, K, rows, seed):
    Mtot = int(sum(rows))
    a, sa = O.quant_1x128(G.bf16_normal((Mtot, K), seed=seed, outlier_frac=1e-3, outlier_scale=30.0), 0, pow2=True)
    bs, sbs = [], []
    for e in range(E):
        b, sb, _, _ = O.quant_128x128(G.bf16_normal((N, K), seed=seed + 10 + e, std=0.02 * (e + 1)), pow2=True)
        bs.append(b)
        sbs.append(sb)
    return a, sa, np.stack(bs), np.stack(sbs), np.repeat(np.arange(E, dtype=np.int32), rows)


@pytest.fixture
def few_cus(dg):
    """Eight compute units: every workgroup walks many work items, and the cost estimate that picks
    between the two tilings (rounds of tiles per compute unit) can favour the paired 256-row tiles, which
    on the whole device these small cases always leave to the 128-row kernel."""
    dg.set_num_sms(8)
    yield
    dg.set_num_sms(0)


def _grouped_call(dg, a, sa, b, sb, m_idx, out, paired):
    """paired: through the mirror, which lets the library pair each expert's 128-row blocks into 256-row
    tiles or hand the call to the 128-row-tile kernel, whichever its cost estimate prefers; otherwise
    the raw C ABI without a work-item list (aligned 256-row tiles, two passes over a tile that holds
    two experts)."""
    ta, tb, tm = G.to_torch_fp8(a), G.to_torch_fp8(b), torch.from_numpy(m_idx).cuda()
    if paired:
        dg.m_grouped_fp8_gemm_nt_contiguous((ta, _e8(sa)), (tb, _e8(sb)), out, tm)
        return
    from paddleformers_amd import _lib

    E, N, K = b.shape
    tsa = _e8(np.ascontiguousarray(sa.T))           # [K/128, Mtot]
    tsb = _e8(sb)
    _lib.call("pf8_grouped_gemm_nt_contiguous_ue8m0", ta.data_ptr(), tsa.data_ptr(), tsa.stride(0), tb.data_ptr(), tsb.data_ptr(),
              E, a.shape[0], N, K, tm.data_ptr(), None, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()


# segments that start in the middle of a 256-row tile (two experts in one aligned tile), segments of
# an odd number of blocks, empty experts, a half tile at the end
@pytest.mark.parametrize("rows", [[128, 256, 0, 128], [0, 0, 384], [128] * 6, [256, 512], [384, 128, 640, 128]])
@pytest.mark.parametrize("paired", [True, False])
@pytest.mark.parametrize("cus", ["all", "few"])
def test_grouped_contiguous_ue8m0_vs_oracle(dg, request, rows, paired, cus):
    if cus == "few":
        request.getfixturevalue("few_cus")
    E, N, K = len(rows), 512, 512
    a, sa, b, sb, m_idx = _grouped_pow2_case(E, N, K, rows, seed=sum(rows) + E)
    Mtot = a.shape[0]
    out = torch.full((Mtot, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    _grouped_call(dg, a, sa, b, sb, m_idx, out, paired)
    exp = O.grouped_gemm_nt_contiguous(a, sa, b, sb, m_idx)
    got = G.from_torch_bf16(out)
    assert G.rel_fro(_bf(got), _bf(exp)) <= BLOCK_FRO
    start = 0
    for e, r in enumerate(rows):
        if r:
            _elementwise_ok(_bf(got[start:start + r]), a[start:start + r], sa[start:start + r], b[e], sb[e], f"expert {e}")
        start += r


# Sixteen K blocks and eight compute units: every persistent workgroup (paired 256-row tiles, and the 128-row-tile
# kernel the list header may hand the call to) runs its copy ring across several tile boundaries, and the aligned
# walk without a list makes a second pass over the tiles in which two experts meet.
@pytest.mark.parametrize("rows", [[256, 0, 640, 128, 384, 512], [128] * 9 + [0, 768], [1024, 896]])
@pytest.mark.parametrize("paired", [True, False])
def test_grouped_contiguous_ue8m0_long_reduction_few_compute_units(dg, few_cus, rows, paired):
    E, N, K = len(rows), 512, 2048
    a, sa, b, sb, m_idx = _grouped_pow2_case(E, N, K, rows, seed=sum(rows) + 7 * E)
    Mtot = a.shape[0]
    out = torch.full((Mtot, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    _grouped_call(dg, a, sa, b, sb, m_idx, out, paired)
    exp = O.grouped_gemm_nt_contiguous(a, sa, b, sb, m_idx)
    got = G.from_torch_bf16(out)
    assert G.rel_fro(_bf(got), _bf(exp)) <= BLOCK_FRO
    start = 0
    for e, r in enumerate(rows):
        if r:
            _elementwise_ok(_bf(got[start:start + r]), a[start:start + r], sa[start:start + r], b[e], sb[e], f"expert {e}")
        start += r


# 640 = two column tiles and a half: the wavefronts of the missing half compute on a copy of the first and
# store nothing.  Through the raw C ABI, so that the block-scaled kernel runs whatever the load: with a
# work-item list (paired 256-row tiles) and without (aligned tiles, two passes where experts meet).
@pytest.mark.parametrize("rows", [[128, 256, 0, 128], [384, 128, 640, 128], [256, 512]])
@pytest.mark.parametrize("with_items", [True, False])
@pytest.mark.parametrize("cus", ["all", "few"])
def test_grouped_contiguous_ue8m0_half_column_tile(dg, request, rows, with_items, cus):
    from paddleformers_amd import _lib

    if cus == "few":
        request.getfixturevalue("few_cus")
    E, N, K = len(rows), 640, 512
    a, sa, b, sb, m_idx = _grouped_pow2_case(E, N, K, rows, seed=sum(rows) + 3 * E)
    Mtot = a.shape[0]
    out = torch.full((Mtot, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    ta, tb, tm = G.to_torch_fp8(a), G.to_torch_fp8(b), torch.from_numpy(m_idx).cuda()
    tsa, tsb = _e8(np.ascontiguousarray(sa.T)), _e8(sb)
    items = dg.build_group_items(tm) if with_items else None
    _lib.call("pf8_grouped_gemm_nt_contiguous_ue8m0", ta.data_ptr(), tsa.data_ptr(), tsa.stride(0), tb.data_ptr(), tsb.data_ptr(),
              E, Mtot, N, K, tm.data_ptr(), items.data_ptr() if with_items else None, out.data_ptr(),
              torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    exp = O.grouped_gemm_nt_contiguous(a, sa, b, sb, m_idx)
    got = G.from_torch_bf16(out)
    assert G.rel_fro(_bf(got), _bf(exp)) <= BLOCK_FRO
    start = 0
    for e, r in enumerate(rows):
        if r:
            _elementwise_ok(_bf(got[start:start + r]), a[start:start + r], sa[start:start + r], b[e], sb[e], f"expert {e}")
        start += r


def _pair_blocks(block_experts):
    """Serial statement of the pairing: consecutive 128-row blocks of one expert two by two, an odd one
    out alone, padding blocks (expert < 0) skipped."""
    items, prev, par = [], -2, 1
    for b, e in enumerate(block_experts):
        if e < 0:
            par, prev = 1, e
            continue
        par = 0 if e != prev else par ^ 1
        if par == 0:
            items.append([b, -1, int(e)])
        else:
            items[-1][1] = b
        prev = e
    return items


# 40 blocks: one block per thread of the list builder; 3000: several blocks per thread; 9000: more blocks
# than the builder keeps in LDS
@pytest.mark.parametrize("nb", [40, 3000, 9000])
def test_build_group_items_pairs_each_experts_blocks(dg, nb):
    rng = np.random.default_rng(nb)
    blocks = []
    e = 0
    while len(blocks) < nb:
        blocks += [e] * int(rng.integers(0, 7))
        if rng.random() < 0.25:
            blocks += [-1] * int(rng.integers(1, 3))
        e += 1
    blocks = np.array(blocks[:nb], np.int32)
    m_idx = torch.from_numpy(np.repeat(blocks, 128)).cuda()
    items = dg.build_group_items(m_idx).cpu().numpy()
    exp = _pair_blocks(blocks)
    assert items[0] == len(exp) and items[1] == nb
    got = items[4:4 + 4 * len(exp)].reshape(-1, 4)[:, :3]
    assert np.array_equal(got, np.array(exp, np.int32).reshape(-1, 3))


@pytest.mark.parametrize("cus", ["all", "few"])
def test_grouped_contiguous_ue8m0_many_small_experts(dg, request, cus):
    """40 experts of 0..5 blocks in Zipf-like disorder, some followed by padding blocks (index -1): every
    routed row is computed with its own expert's weights and every padding row is left alone."""
    if cus == "few":
        request.getfixturevalue("few_cus")
    rng = np.random.default_rng(12)
    E, N, K = 40, 256, 384
    rows = [int(128 * rng.integers(0, 6)) for _ in range(E)]
    a, sa, b, sb, m_idx = _grouped_pow2_case(E, N, K, rows, seed=77)
    pad = np.zeros(len(m_idx), bool)
    start = 0
    for e, r in enumerate(rows):
        if r >= 256 and rng.random() < 0.4:
            pad[start + r - 128:start + r] = True         # the expert's last block is padding
        start += r
    m_idx = m_idx.copy()
    m_idx[pad] = -1
    out = torch.full((len(m_idx), N), 7.0, dtype=torch.bfloat16, device="cuda")
    _grouped_call(dg, a, sa, b, sb, m_idx, out, True)
    got = G.from_torch_bf16(out)
    seven = O.f32_to_bf16_bits(np.full((1,), 7.0, np.float32))[0]
    assert (got[pad] == seven).all()
    init = np.full(got.shape, seven, np.uint16)
    exp = O.grouped_gemm_nt_contiguous(a, sa, b, sb, m_idx, out=init)
    assert G.rel_fro(_bf(got[~pad]), _bf(exp[~pad])) <= BLOCK_FRO


@pytest.mark.parametrize("paired", [True, False])
def test_grouped_contiguous_ue8m0_negative_index_skips_rows(dg, paired):
    """Padding rows (index -1) are left untouched whichever half of a 256-row tile they fill."""
    E, N, K = 3, 256, 384
    rows = [256, 256, 256]
    a, sa, b, sb, m_idx = _grouped_pow2_case(E, N, K, rows, seed=5)
    m_idx[128:256] = -1       # second half of tile 0
    m_idx[256:384] = -1       # first half of tile 1
    m_idx[512:768] = -1       # all of tile 2
    out = torch.full((768, N), 7.0, dtype=torch.bfloat16, device="cuda")
    _grouped_call(dg, a, sa, b, sb, m_idx, out, paired)
    got = G.from_torch_bf16(out)
    seven = O.f32_to_bf16_bits(np.full((1,), 7.0, np.float32))[0]
    for lo, hi, e in [(0, 128, 0), (384, 512, 1)]:
        exp = O.gemm_nt(a[lo:hi], sa[lo:hi], b[e], sb[e])
        assert G.rel_fro(_bf(got[lo:hi]), _bf(exp)) <= BLOCK_FRO
    for lo, hi in [(128, 384), (512, 768)]:
        assert (got[lo:hi] == seven).all()


def test_ue8m0_gemms_at_config3_size_agree_with_the_fp32_scale_kernels(dg):
    """Full forward shapes of config 3 (10240 rows, 8 experts of 1280): the block-scaled kernel and the
    fp32-scale kernel see the same pow2 scales, so their bf16 outputs differ by rounding flips only."""
    from paddleformers_amd import functional as F

    E, rows, H, I2 = 8, 1280, 7168, 4096
    Mtot = E * rows
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn((Mtot, H), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    w = (torch.randn((E, I2, H), generator=gen, device="cuda", dtype=torch.float32) * 0.02).to(torch.bfloat16)
    xq, xs = F.fp8_quant_blockwise(x, output_scale_transpose=True, quant_method="1x128", input_transpose=False, using_pow2_scale=True)
    wq, ws = F.fused_stack_transpose_quant([w[e] for e in range(E)], transpose=False, using_pow2_scale=True)
    wq, ws = wq.view(E, I2, H), ws.view(E, I2 // 128, H // 128)
    m_idx = torch.arange(E, dtype=torch.int32, device="cuda").repeat_interleave(rows)
    xs_l = xs.t() if tuple(xs.shape) == (H // 128, Mtot) else xs         # logical [Mtot, H/128]
    ref = torch.empty((Mtot, I2), dtype=torch.bfloat16, device="cuda")
    dg.m_grouped_fp8_gemm_nt_contiguous((xq, xs_l), (wq, ws), ref, m_idx)
    out = torch.empty_like(ref)
    dg.m_grouped_fp8_gemm_nt_contiguous((xq, F.scales_to_ue8m0(xs_l)), (wq, F.scales_to_ue8m0(ws)), out, m_idx)
    d = (out.float() - ref.float()).norm() / ref.float().norm()
    assert d.item() <= 3e-4, d.item()
    # dense call on one expert's segment: same kernel family, same numbers as the grouped call
    one = torch.empty((rows, I2), dtype=torch.bfloat16, device="cuda")
    sl = slice(3 * rows, 4 * rows)
    dg.fp8_gemm_nt((xq[sl], F.scales_to_ue8m0(xs_l[sl].contiguous())), (wq[3], F.scales_to_ue8m0(ws[3])), one)
    assert torch.equal(one.view(torch.int16), out[sl].view(torch.int16))


# N = 2816: the up+gate GEMM; N = 1408 (five column tiles and a half): the dgrad GEMM of the down projection
@pytest.mark.parametrize("N", [2816, 1408])
def test_ue8m0_grouped_gemm_at_config5_size_agrees_with_the_fp32_scale_kernel(dg, N):
    """128 experts with a Zipf(1.0) load over 131072 routed rows (segments of 2..190 blocks, 1083 blocks in
    all): here the cost estimate picks the paired 256-row tiles on the whole device, and the list builder
    walks two blocks per thread."""
    zipf_counts = G.zipf_counts
    from paddleformers_amd import deep_gemm as DG
    from paddleformers_amd import functional as F

    E, H = 128, 4096
    assert DG._ue8m0_kernel_shape(138624, N, H, E)
    _, padded = zipf_counts(131072, E, 1.0, seed=5, n_empty=0)
    rows = [int(r) for r in padded]
    Mtot = sum(rows)
    gen = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn((Mtot, H), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    xq, xs = F.fp8_quant_blockwise(x, output_scale_transpose=True, quant_method="1x128", input_transpose=False, using_pow2_scale=True)
    del x
    wq = torch.empty((E, N, H), dtype=torch.float8_e4m3fn, device="cuda")
    ws = torch.empty((E, N // 128, H // 128), dtype=torch.float32, device="cuda")
    for e in range(E):
        w = (torch.randn((N, H), generator=gen, device="cuda", dtype=torch.float32) * 0.02).to(torch.bfloat16)
        q, s_ = F.fused_stack_transpose_quant([w], transpose=False, using_pow2_scale=True)
        wq[e], ws[e] = q.view(N, H), s_.view(N // 128, H // 128)
    m_idx = torch.repeat_interleave(torch.arange(E, dtype=torch.int32), torch.tensor(rows)).cuda()
    xs_l = xs.t() if tuple(xs.shape) == (H // 128, Mtot) else xs
    ref = torch.empty((Mtot, N), dtype=torch.bfloat16, device="cuda")
    dg.m_grouped_fp8_gemm_nt_contiguous((xq, xs_l), (wq, ws), ref, m_idx)
    out = torch.full_like(ref, float("nan"))
    dg.m_grouped_fp8_gemm_nt_contiguous((xq, F.scales_to_ue8m0(xs_l)), (wq, F.scales_to_ue8m0(ws)), out, m_idx)
    items = dg.build_group_items(m_idx).cpu().numpy()
    assert items[1] == Mtot // 128 and items[0] == sum((r // 128 + 1) // 2 for r in rows)
    num = den = 0.0
    for lo in range(0, Mtot, 16384):      # in slices: the fp32 copies of two 780 MB outputs are not needed at once
        a, b = out[lo:lo + 16384].float(), ref[lo:lo + 16384].float()
        num += float((a - b).pow(2).sum())
        den += float(b.pow(2).sum())
    assert (num / den) ** 0.5 <= 3e-4
