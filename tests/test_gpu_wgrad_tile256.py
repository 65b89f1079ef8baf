"""GPU tests of the grouped weight gradient's second kernel (256x256 accumulator tile, power-of-two scales inside the
block-scaled MFMA), through the C ABI.

`pf8_grouped_wgrad_pow2` hands the experts whose reduction axis is long to that kernel and the others to the 128x128-tile
kernel.  Both accumulate the same 128-deep blocks with the same instruction in the same order, so the bar is bit identity
between the two routes (the self-test hook switches the second kernel off), on top of the oracle comparison the
128x128-tile route already has; one case also goes straight to the oracle's weight-gradient GEMM
(transformers/fp8_utils.py:1117-1129, the loop the grouped launch replaces)."""
import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

F32_FRO_MFMA_ACC = 1e-4   # fp32 outputs vs the oracle when the running sum stays inside the matrix pipe


@pytest.fixture()
def knobs():
    """Sets the compute-unit budget and the routing threshold for one test and restores both."""
    from paddleformers_amd import _lib

    L = _lib.lib()
    state = {"cus": L.pf8_get_num_cus(), "blocks": L.pf8_debug_set_wgrad_tile256_min_blocks(6)}

    def set_(cus, blocks):
        L.pf8_set_num_cus(cus)
        L.pf8_debug_set_wgrad_tile256_min_blocks(blocks)

    yield set_
    L.pf8_set_num_cus(state["cus"])
    L.pf8_debug_set_wgrad_tile256_min_blocks(state["blocks"])


def _operands(Kin, N, rows, seed):
    from paddleformers_amd import functional as F8

    M = sum(rows)
    x = G.to_torch_bf16(G.bf16_normal((M, Kin), seed=seed))
    d = G.to_torch_bf16(G.bf16_normal((M, N), seed=seed + 1, std=3.0))
    return F8.fused_transpose_split_quant(x, None, rows, True), F8.fused_transpose_split_quant(d, None, rows, True)


# (Kin, N, rows per expert, compute-unit budget, blocks from which an expert takes the 256x256 tile)
CASES = [
    # eight compute units: the three long experts' 24 tiles fill them, the short and the empty expert stay behind
    (512, 1024, [512, 0, 1536, 128, 640], 8, 4),
    # both axes end in a half tile (Kin = 2.5 tiles, N = 1.5 tiles)
    (640, 384, [1024, 512, 0, 768], 8, 4),
    # every expert long: the 128x128-tile kernel is not launched at all
    (512, 512, [768, 1024], 8, 4),
    # 256 experts (the most one call takes), one 256x256 tile each: most XCDs get an empty slice of every expert
    (256, 256, [512] * 256, 8, 4),
    # the whole device, shapes of the MoE node's two weight gradients (I = 1408, H = 4096)
    (1408, 4096, [2048, 1024, 128, 3072, 0, 512, 1536], 0, 8),
    (4096, 2816, [2048, 1024, 128, 3072], 0, 8),
]


@pytest.mark.parametrize("accumulate", [True, False])
@pytest.mark.parametrize("Kin,N,rows,cus,blocks", CASES)
def test_both_kernels_of_the_grouped_weight_gradient_give_the_same_bits(knobs, Kin, N, rows, cus, blocks, accumulate):
    from paddleformers_amd import functional as F8

    (a_t, sa_t), (b_t, sb_t) = _operands(Kin, N, rows, seed=11)
    base = torch.randn((len(rows), Kin, N), device="cuda")
    outs = []
    for threshold in (0, blocks):          # 0: every expert on the 128x128-tile kernel
        knobs(cus, threshold)
        g = base.clone()
        F8.grouped_wgrad(a_t, sa_t, b_t, sb_t, g, accumulate=accumulate, scales_pow2=True)
        outs.append(g)
    assert torch.equal(outs[0], outs[1])
    for e, r in enumerate(rows):
        if r == 0:
            assert torch.equal(outs[1][e], base[e] if accumulate else torch.zeros_like(base[e]))


def test_long_experts_against_the_oracle(knobs):
    from paddleformers_amd import functional as F8

    Kin, N, rows = 512, 1024, [1536, 128, 640]
    (a_t, sa_t), (b_t, sb_t) = _operands(Kin, N, rows, seed=21)
    knobs(8, 4)
    out = torch.full((len(rows), Kin, N), float("nan"), device="cuda")
    F8.grouped_wgrad(a_t, sa_t, b_t, sb_t, out, accumulate=False, scales_pow2=True)
    for e in range(len(rows)):
        exp = O.gemm_nt_1d1d_f32(G.from_torch_fp8(a_t[e]), sa_t[e].cpu().numpy(), G.from_torch_fp8(b_t[e]), sb_t[e].cpu().numpy())
        assert G.rel_fro(out[e].cpu().numpy(), exp) <= F32_FRO_MFMA_ACC, f"expert {e}"


def test_launches_that_overlap_on_two_streams_draw_from_separate_counters(knobs):
    """The kernel hands out tiles through per-launch ticket counters; two launches in flight at once must not share them."""
    from paddleformers_amd import functional as F8

    Kin, N, rows = 512, 1024, [1536, 640, 512, 1024]
    (a_t, sa_t), (b_t, sb_t) = _operands(Kin, N, rows, seed=31)
    base = torch.randn((len(rows), Kin, N), device="cuda")
    knobs(8, 0)
    ref = base.clone()
    F8.grouped_wgrad(a_t, sa_t, b_t, sb_t, ref, accumulate=True, scales_pow2=True)
    knobs(8, 4)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [base.clone(), base.clone()]
    torch.cuda.synchronize()
    for _ in range(3):
        for s, o in zip(streams, outs):
            with torch.cuda.stream(s):
                o.copy_(base)
                F8.grouped_wgrad(a_t, sa_t, b_t, sb_t, o, accumulate=True, scales_pow2=True)
    torch.cuda.synchronize()
    for o in outs:
        assert torch.equal(o, ref)
    # 70 launches in a row pass through every counter slot more than once: each must have been left clear
    o = outs[0]
    for _ in range(70):
        o.copy_(base)
        F8.grouped_wgrad(a_t, sa_t, b_t, sb_t, o, accumulate=True, scales_pow2=True)
    assert torch.equal(o, ref)


def test_routing_threshold_hook_returns_the_previous_setting():
    from paddleformers_amd import _lib

    L = _lib.lib()
    prev = L.pf8_debug_set_wgrad_tile256_min_blocks(9)
    assert L.pf8_debug_set_wgrad_tile256_min_blocks(prev) == 9
