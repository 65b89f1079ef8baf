"""GPU parity tests of the GEMMs that read FRAGMENT-MAJOR weights (`pf8_weight_to_fragment_major`,
`pf8_gemm_nt_fm`, `pf8_grouped_gemm_nt_contiguous_fm`) through the deep_gemm-named mirror, i.e. through the C ABI.

The byte order is pinned by un-permuting on the host with the formula the header states; the GEMMs are compared with
the CPU oracle at the bars of tests/test_gpu_gemm.py and with the kernels that read the plain weight: same scale
factors and order of the K blocks, but a K block's product comes from two chained 32x32x64 instructions instead of one
16x16x128, so the two agree to the matrix pipe's own precision (a few 1e-6 of sum|a||b| per block), not to the bit."""
import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

REL_FRO = 1e-3
BLOCK_FRO = 6e-4
SAME_MATH_FRO = 2e-4   # against the plain-weight kernel: bf16 roundings that flip on a difference in the matrix pipe's last bits


@pytest.fixture(scope="module")
def dg():
    from paddleformers_amd import _lib, deep_gemm

    _lib.lib()
    return deep_gemm


def _fm_reference(w):
    """[E, N, K] bytes -> the fragment-major order, by the formula of include/pf8.h, in numpy."""
    E, N, K = w.shape
    v = w.reshape(E, N // 64, 2, 32, K // 128, 2, 2, 2, 16)     # e, n64, pf, x, kb, kh, hh, h, byte
    v = v.transpose(0, 1, 4, 2, 5, 7, 6, 3, 8)                   # e, n64, kb, pf, kh, h, hh, x, byte  (lane = 32 hh + x)
    return np.ascontiguousarray(v).reshape(E, N, K)


@pytest.mark.parametrize("E,N,K", [(1, 64, 128), (3, 256, 512), (2, 192, 1408)])
def test_fragment_major_byte_order(dg, E, N, K):
    rng = np.random.default_rng(E * N + K)
    w = rng.integers(0, 256, size=(E, N, K), dtype=np.uint8)
    fm = dg.to_fragment_major(G.to_torch_fp8(w))
    assert fm.shape == (E, N, K)
    got = fm.data.view(torch.uint8).cpu().numpy()
    assert (got == _fm_reference(w)).all()
    # a 2-D weight is one expert
    fm2 = dg.to_fragment_major(G.to_torch_fp8(w[0]))
    assert (fm2.data.view(torch.uint8).cpu().numpy() == _fm_reference(w[:1])[0]).all()
    with pytest.raises(ValueError):
        dg.to_fragment_major(G.to_torch_fp8(w[:, :32]))


def _dense_case(M, N, K, seed):
    a, sa = O.quant_1x128(G.bf16_normal((M, K), seed=seed, outlier_frac=1e-3, outlier_scale=30.0), 0)
    b, sb, _, _ = O.quant_128x128(G.bf16_normal((N, K), seed=seed + 1, std=0.02, outlier_frac=5e-4, outlier_scale=50.0))
    return a, sa, b, sb


@pytest.mark.parametrize("M,N,K", [(128, 256, 384), (128, 256, 512), (384, 512, 1024), (256, 768, 2048), (1280, 256, 640), (256, 256, 1408),
                                   (256, 384, 512), (384, 1408, 640), (128, 640, 384)])          # the last three: a half last column tile
@pytest.mark.parametrize("lay", [0, 1])
def test_dense_fragment_major_against_oracle_and_plain_kernel(dg, M, N, K, lay):
    a, sa, b, sb = _dense_case(M, N, K, seed=M + N + K)
    ta, tb = G.to_torch_fp8(a), G.to_torch_fp8(b)
    tsa = torch.from_numpy(np.ascontiguousarray(sa.T)).cuda().t() if lay else torch.from_numpy(sa).cuda()
    tsb = torch.from_numpy(sb).cuda()
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    dg.fp8_gemm_nt((ta, tsa), (dg.to_fragment_major(tb), tsb), out)
    got = G.from_torch_bf16(out)
    ref = O.gemm_nt(a, sa, b, sb, dequant_ref=True)
    blk = O.gemm_nt(a, sa, b, sb)
    assert G.rel_fro(O.bf16_bits_to_f32(got), O.bf16_bits_to_f32(ref)) <= REL_FRO
    assert G.rel_fro(O.bf16_bits_to_f32(got), O.bf16_bits_to_f32(blk)) <= BLOCK_FRO
    plain = torch.empty_like(out)
    dg.fp8_gemm_nt((ta, tsa), (tb, tsb), plain)
    assert G.rel_fro(out.float().cpu().numpy(), plain.float().cpu().numpy()) <= SAME_MATH_FRO


def test_dense_fragment_major_exact_integers(dg):
    """Small-integer codes and power-of-two scales: every product and sum is exact, so the output is known exactly; a
    misplaced fragment, row permutation or scale shows as a wrong integer."""
    M, N, K = 256, 512, 1024
    rng = np.random.default_rng(7)
    av = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    bv = rng.integers(-2, 3, size=(N, K)).astype(np.float32)
    a, b = O.e4m3_encode_array(av), O.e4m3_encode_array(bv)
    sa = (2.0 ** rng.integers(-2, 3, size=(M, K // 128))).astype(np.float32)
    sb = (2.0 ** rng.integers(-2, 3, size=(N // 128, K // 128))).astype(np.float32)
    exact = (av * np.repeat(sa, 128, axis=1)) @ (bv * np.repeat(np.repeat(sb, 128, axis=0), 128, axis=1)).T
    out = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    dg.fp8_gemm_nt((G.to_torch_fp8(a), torch.from_numpy(sa).cuda()), (dg.to_fragment_major(G.to_torch_fp8(b)), torch.from_numpy(sb).cuda()), out)
    want = O.f32_to_bf16_bits(exact.astype(np.float32))
    assert (G.from_torch_bf16(out) == want).all()


def _grouped_case(E, N, K, blocks, seed):
    """blocks: list of (expert or -1, number of 128-row tiles)."""
    Mtot = 128 * sum(n for _, n in blocks)
    a, sa = O.quant_1x128(G.bf16_normal((Mtot, K), seed=seed, outlier_frac=1e-3, outlier_scale=30.0), 0)
    bs, sbs = zip(*[O.quant_128x128(G.bf16_normal((N, K), seed=seed + 10 + e, std=0.02, outlier_frac=5e-4, outlier_scale=50.0))[:2]
                    for e in range(E)])
    m_idx = np.concatenate([np.full(128 * n, e, dtype=np.int32) for e, n in blocks])
    return a, sa, np.stack(bs), np.stack(sbs), m_idx


@pytest.mark.parametrize("K,blocks", [
    (512, [(0, 1), (2, 3), (-1, 1), (1, 2)]),
    (384, [(1, 2), (-1, 1), (0, 1), (3, 4)]),
    (1024, [(3, 13), (-1, 1), (1, 1), (2, 25), (-1, 2), (0, 2), (0, 1)]),
    (896, [(e % 4, 1 + (e * 5) % 4) for e in range(12)]),
    (512, [(e % 4, 1 + (e * 7) % 3) for e in range(30)]),
])
@pytest.mark.parametrize("lay", [0, 1])
@pytest.mark.parametrize("cus", [0, 16])
@pytest.mark.parametrize("N", [512, 384])
def test_grouped_fragment_major_against_oracle_and_plain_kernel(dg, K, blocks, lay, cus, N):
    E = 4
    a, sa, b, sb, m_idx = _grouped_case(E, N, K, blocks, seed=K + len(blocks))
    Mtot = a.shape[0]
    ta, tb = G.to_torch_fp8(a), G.to_torch_fp8(b)
    tsa = torch.from_numpy(np.ascontiguousarray(sa.T)).cuda().t() if lay else torch.from_numpy(sa).cuda()
    tsb, tm = torch.from_numpy(sb).cuda(), torch.from_numpy(m_idx).cuda()
    out = torch.full((Mtot, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    plain = torch.full((Mtot, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    dg.set_num_sms(cus)
    try:
        dg.m_grouped_fp8_gemm_nt_contiguous((ta, tsa), (dg.to_fragment_major(tb), tsb), out, tm)
        dg.m_grouped_fp8_gemm_nt_contiguous((ta, tsa), (tb, tsb), plain, tm)
    finally:
        dg.set_num_sms(0)
    # padding tiles are left untouched by both kernels
    valid = torch.from_numpy(m_idx >= 0).cuda()
    assert torch.isnan(out[~valid].float()).all()
    assert G.rel_fro(out[valid].float().cpu().numpy(), plain[valid].float().cpu().numpy()) <= SAME_MATH_FRO
    exp = O.grouped_gemm_nt_contiguous(a, sa, b, sb, m_idx)
    got = G.from_torch_bf16(out)
    v = m_idx >= 0
    assert G.rel_fro(O.bf16_bits_to_f32(got[v]), O.bf16_bits_to_f32(exp[v])) <= BLOCK_FRO


def test_fragment_major_rejects_other_shapes_and_scales(dg):
    a, sa, b, sb = _dense_case(128, 256, 512, seed=3)
    ta, tb = G.to_torch_fp8(a), G.to_torch_fp8(b)
    tsa, tsb = torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda()
    fm = dg.to_fragment_major(tb)
    assert dg.fragment_major_supported(128, 256, 512) and dg.fragment_major_supported(128, 256, 384)
    assert dg.fragment_major_supported(128, 384, 512) and not dg.fragment_major_supported(128, 320, 512)
    assert not dg.fragment_major_supported(128, 128, 512) and not dg.fragment_major_supported(128, 256, 256)
    assert not dg.fragment_major_supported(100, 256, 512)
    with pytest.raises(ValueError):                             # K = 256: fewer than three K blocks
        dg.fp8_gemm_nt((ta[:, :256].contiguous(), tsa[:, :2].contiguous()),
                       (dg.to_fragment_major(tb[:, :256].contiguous()), tsb[:, :2].contiguous()),
                       torch.empty((128, 256), dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):                             # UE8M0 scales go to the block-scaled kernel, which reads plain weights
        dg.fp8_gemm_nt((ta, tsa.to(torch.uint8)), (fm, tsb.to(torch.uint8)), torch.empty((128, 256), dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):                             # the weight-gradient recipe has no fragment-major form
        dg.fp8_gemm_nt((ta, tsa), (fm, tsb), torch.empty((128, 256), dtype=torch.float32, device="cuda"), recipe=(1, 1, 128))
