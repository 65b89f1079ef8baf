"""GPU tests of the unzip that copies no row: `moe_permute(..., do_gather=False)` hands out the source token of every
expert-sorted row, and the two consumers of the unzipped FP8 tokens (the up+gate grouped GEMM on a fragment-major weight,
the transposed quantizer of the weight gradient) read the tokens through that map.

The map is pinned by the CPU oracle's moe_permute (the inverse of its row map); the consumers must equal, to the bit, the
same kernels run on the rows `moe_permute` copies out, which the oracle pins in tests/test_gpu_permute.py,
tests/test_gpu_gemm_fm.py and tests/test_gpu_quant.py."""
import types

import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G
from tests.test_gpu_permute import routing

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def F():
    from paddleformers_amd import _lib
    from paddleformers_amd import functional as F8

    _lib.lib()
    return F8


def _tokens(T, H, seed):
    """Quantized tokens as the dispatcher hands them over: e4m3 codes and 1x128 scales of a bf16 matrix."""
    q, s = O.quant_1x128(G.bf16_normal((T, H), seed=seed, outlier_frac=1e-3, outlier_scale=30.0), 0)
    return q, s


def _both(F, q, s, rm, probs, E, counts, align=128):
    trm, tpr = torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
    tq, ts = G.to_torch_fp8(q), torch.from_numpy(s).cuda()
    copied = F.moe_permute(tq, ts, trm, tpr, E, counts, align)
    mapped = F.moe_permute(tq, ts, trm, tpr, E, counts, align, do_gather=False)
    return copied, mapped


@pytest.mark.parametrize("T,H,topk,E,align", [(37, 256, 4, 8, 128), (300, 1408, 2, 5, 128), (9, 128, 1, 3, 16), (1, 128, 3, 4, 128),
                                              (4100, 128, 8, 16, 128)])
def test_source_map_against_oracle_and_copy(F, T, H, topk, E, align):
    rm, probs, counts = routing(T, topk, E, seed=T + H)
    q, s = _tokens(T, H, seed=T)
    ox, orow, op, osc = O.moe_permute(q, s, rm, probs, E, counts, align)
    (cx, crow, cp, cs), (g, grow, gp, gs) = _both(F, q, s, rm, probs, E, counts, align)
    assert gs is None and isinstance(g, F.GatheredRows) and tuple(g.shape) == tuple(cx.shape)
    # the inverse of the oracle's row map; every other row is padding
    want = np.full(ox.shape[0], -1, np.int32)
    t_idx, e_idx = np.nonzero(orow >= 0)
    want[orow[t_idx, e_idx]] = t_idx
    assert (g.src_row.cpu().numpy() == want).all(), "source rows"
    assert (grow.cpu().numpy() == orow).all() and (gp.cpu().numpy() == op).all()
    rows, scales = g.materialize()
    assert (G.from_torch_fp8(rows) == ox).all() and (scales.cpu().numpy() == osc).all()
    assert torch.equal(rows.view(torch.uint8), cx.view(torch.uint8)) and torch.equal(scales, cs) and torch.equal(gp, cp)
    # a slice of gathered rows is the slice of the map
    if ox.shape[0] >= 32:
        part = g[16:32]
        assert tuple(part.shape) == (16, H) and torch.equal(part.materialize()[0].view(torch.uint8), cx[16:32].view(torch.uint8))
    with pytest.raises(TypeError):
        g[::2]


def test_source_map_flags_counts_that_disagree_with_the_routing(F):
    T, H, topk, E = 200, 128, 2, 4
    rm, probs, counts = routing(T, topk, E, seed=9, drop=0.0)
    q, s = _tokens(T, H, seed=2)
    tq, ts, trm, tpr = G.to_torch_fp8(q), torch.from_numpy(s).cuda(), torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
    F.moe_permute_check()
    short = list(counts)
    short[1] -= 3
    with pytest.raises(ValueError):
        F.moe_permute(tq, ts, trm, tpr, E, short, 128, do_gather=False, validate=True)
    long = list(counts)
    long[2] += 5
    g, _, gp, _ = F.moe_permute(tq, ts, trm, tpr, E, long, 128, do_gather=False)
    with pytest.raises(ValueError):
        F.moe_permute_check()
    cx, _, cp, cs = F.moe_permute(tq, ts, trm, tpr, E, long, 128)
    with pytest.raises(ValueError):
        F.moe_permute_check()
    # the rows of the overstated count read as zeros, as the copy writes them
    rows, scales = g.materialize()
    assert torch.equal(rows.view(torch.uint8), cx.view(torch.uint8)) and torch.equal(scales, cs) and torch.equal(gp, cp)


def test_source_map_of_bf16_tokens_and_their_per_token_quantization(F):
    """Gradient tokens: bf16 rows behind the map; quantizing the T tokens gives every copy the bytes and scales that
    quantizing the copied rows gives (the 1x128 rule is per row)."""
    T, H, topk, E = 333, 512, 3, 5
    rm, probs, counts = routing(T, topk, E, seed=12)
    bits = G.bf16_normal((T, H), seed=13, outlier_frac=1e-3, outlier_scale=50.0)
    tx, trm, tpr = G.to_torch_bf16(bits), torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
    cx, crow, cp, _ = F.moe_permute(tx, None, trm, tpr, E, counts, 128)
    g, grow, gp, gs = F.moe_permute(tx, None, trm, tpr, E, counts, 128, do_gather=False)
    assert gs is None and g.scale is None and g.dtype == torch.bfloat16 and torch.equal(grow, crow) and torch.equal(gp, cp)
    assert torch.equal(g.materialize().view(torch.int16), cx.view(torch.int16))
    for pow2 in (False, True):
        cq, cs = F.fp8_quant_blockwise(cx, quant_method="1x128", using_pow2_scale=pow2)
        gq = g.quantize(pow2)
        assert gq.dtype == F.FP8 and gq.quantize(pow2) is gq
        rows, scales = gq.materialize()
        live = (g.src_row >= 0)
        assert torch.equal(rows.view(torch.uint8), cq.view(torch.uint8))
        assert torch.equal(scales[live], cs[live])          # (the copy gives a padding row the scale of an all-zero tile, 1)
        assert (scales[~live] == 0).all() and (cs[~live] == 1).all()


def _weights(E, N, K, seed):
    bs, sbs = zip(*[O.quant_128x128(G.bf16_normal((N, K), seed=seed + e, std=0.02, outlier_frac=5e-4, outlier_scale=50.0))[:2] for e in range(E)])
    return np.stack(bs), np.stack(sbs)


@pytest.mark.parametrize("T,K,N,topk,E", [(300, 512, 512, 2, 5), (1000, 384, 256, 3, 4), (700, 1408, 768, 4, 8), (90, 1024, 512, 1, 6),
                                         (400, 512, 640, 2, 3)])
@pytest.mark.parametrize("cus", [0, 16])
def test_grouped_gemm_reads_through_the_source_map(F, T, K, N, topk, E, cus):
    from paddleformers_amd import deep_gemm as dg

    rm, probs, counts = routing(T, topk, E, seed=T + K, drop=0.15)
    q, s = _tokens(T, K, seed=K)
    (cx, _, _, cs), (g, _, _, _) = _both(F, q, s, rm, probs, E, counts)
    b, sb = _weights(E, N, K, seed=T)
    wfm, tsb = dg.to_fragment_major(G.to_torch_fp8(b)), torch.from_numpy(sb).cuda()
    padded = [(c + 127) // 128 * 128 for c in counts]
    m_idx = torch.from_numpy(np.repeat(np.arange(E, dtype=np.int32), padded)).cuda()
    Mtot = sum(padded)
    out_c = torch.full((Mtot, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    out_g = torch.full((Mtot, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    dg.set_num_sms(cus)
    try:
        dg.m_grouped_fp8_gemm_nt_contiguous((cx, cs), (wfm, tsb), out_c, m_idx)
        dg.m_grouped_fp8_gemm_nt_contiguous((g, None), (wfm, tsb), out_g, m_idx)
    finally:
        dg.set_num_sms(0)
    assert not torch.isnan(out_c.float()).any()
    assert torch.equal(out_g.view(torch.int16), out_c.view(torch.int16))
    # padding rows come out as zeros from both
    pad = g.src_row < 0
    assert pad.any() and (out_g[pad].float() == 0).all()
    # against the oracle, at the bar of the fragment-major kernel
    ox, _, _, osc = O.moe_permute(q, s, rm, probs, E, counts, 128)
    exp = O.grouped_gemm_nt_contiguous(ox, osc, b, sb, m_idx.cpu().numpy())
    assert G.rel_fro(O.bf16_bits_to_f32(G.from_torch_bf16(out_g)), O.bf16_bits_to_f32(exp)) <= 6e-4


def test_grouped_gemm_through_the_map_rejects_what_it_cannot_read(F):
    from paddleformers_amd import deep_gemm as dg

    T, K, N, E = 256, 512, 256, 2
    rm, probs, counts = routing(T, 1, E, seed=1, drop=0.0)
    q, s = _tokens(T, K, seed=3)
    _, (g, _, _, _) = _both(F, q, s, rm, probs, E, counts)
    b, sb = _weights(E, N, K, seed=5)
    tb, tsb = G.to_torch_fp8(b), torch.from_numpy(sb).cuda()
    Mtot = g.shape[0]
    out = torch.empty((Mtot, N), dtype=torch.bfloat16, device="cuda")
    m_idx = torch.zeros(Mtot, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):                 # plain weight
        dg.m_grouped_fp8_gemm_nt_contiguous((g, None), (tb, tsb), out, m_idx)
    with pytest.raises(ValueError):                 # scales come with the rows
        dg.m_grouped_fp8_gemm_nt_contiguous((g, g.scale), (dg.to_fragment_major(tb), tsb), out, m_idx)
    with pytest.raises(ValueError):                 # the dense GEMM does not read gathered rows
        dg.fp8_gemm_nt((g, None), (dg.to_fragment_major(tb[0]), tsb[0]), out)


@pytest.mark.parametrize("T,K,topk,E", [(300, 512, 2, 5), (1000, 128, 3, 4), (260, 1408, 4, 8)])
@pytest.mark.parametrize("pow2", [True, False])
@pytest.mark.parametrize("bf16", [False, True])
def test_transposed_quantizer_reads_through_the_source_map(F, T, K, topk, E, pow2, bf16):
    rm, probs, counts = routing(T, topk, E, seed=T + K + 1, drop=0.1)
    padded = [(c + 127) // 128 * 128 for c in counts]
    if bf16:
        tx = G.to_torch_bf16(G.bf16_normal((T, K), seed=K + 9, outlier_frac=1e-3, outlier_scale=30.0))
        trm, tpr = torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
        cx, cs = F.moe_permute(tx, None, trm, tpr, E, counts, 128)[0], None
        g = F.moe_permute(tx, None, trm, tpr, E, counts, 128, do_gather=False)[0]
    else:
        q, s = _tokens(T, K, seed=K + 7)
        (cx, _, _, cs), (g, _, _, _) = _both(F, q, s, rm, probs, E, counts)
    qc, sc = F.fused_transpose_split_quant(cx, cs, padded, pow2)
    qg, sg = F.fused_transpose_split_quant(g, None, padded, pow2)
    assert len(qc) == len(qg) == E
    for e in range(E):
        assert qc[e].shape == qg[e].shape and sc[e].shape == sg[e].shape
        assert torch.equal(qc[e].view(torch.uint8), qg[e].view(torch.uint8)), f"expert {e} bytes"
        assert torch.equal(sc[e], sg[e]), f"expert {e} scales"
    if not bf16:
        with pytest.raises(ValueError):
            F.fused_transpose_split_quant(g, g.scale, padded, pow2)


@pytest.mark.parametrize("recompute", [False, True])
def test_expert_mlp_node_on_gathered_rows_equals_the_node_on_copied_rows(F, recompute):
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode, fp8_quant_weight
    from tests.test_gpu_fusion_mlp_node import _fresh_experts
    from tests.test_gpu_moe_layer import _layer

    T, H, I, E, topk = 500, 512, 256, 6, 3
    rm, probs, counts, w1, w2, _, x, dy = _layer(T, H, I, E, topk, seed=77)
    tq, ts = F.fp8_quant_blockwise(G.to_torch_bf16(x), quant_method="1x128")
    trm, tpr = torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
    cx, _, cp, cs = F.moe_permute(tq, ts, trm, tpr, E, counts, 128)
    g, _, gp, _ = F.moe_permute(tq, ts, trm, tpr, E, counts, 128, do_gather=False)
    padded = [(c + 127) // 128 * 128 for c in counts]
    # the gradient arrives as tokens too (ZipNode.backward): copied rows for the one node, the map for the other
    tg = torch.randn((T, H), generator=torch.Generator(device="cuda").manual_seed(6), device="cuda").to(torch.bfloat16)
    grad = F.moe_permute(tg, None, trm, tpr, E, counts, 128)[0]
    grad_map = F.moe_permute(tg, None, trm, tpr, E, counts, 128, do_gather=False)[0]
    results = []
    for rows in ((cx, cs), g):
        experts = _fresh_experts(w1, w2)
        fp8_quant_weight([e.w1 for e in experts], [e.w2 for e in experts], batch_mode=True)      # the per-step FP8 weight cache
        node = FP8GroupGemmMlpFunctionNode(types.SimpleNamespace(experts=experts), recompute_fwd_gate_up=recompute)
        o3 = node.forward(rows, cp, padded)
        if rows is g:
            assert isinstance(node.input_fp8, F.GatheredRows) and node.input_scale is None     # nothing was copied
        dx, pg = node.backward(grad_map if rows is g else grad, cp, padded)
        results.append((o3, dx, pg, [e.w1.main_grad for e in experts], [e.w2.main_grad for e in experts]))
    a, b = results
    assert torch.equal(a[0].view(torch.int16), b[0].view(torch.int16)) and torch.equal(a[1].view(torch.int16), b[1].view(torch.int16))
    assert torch.equal(a[2], b[2])
    for ga, gb in zip(a[3] + a[4], b[3] + b[4]):
        assert (ga is None) == (gb is None) and (ga is None or torch.equal(ga, gb))


@pytest.mark.parametrize("fp8_dispatch", [True, False])
def test_fusion_mlp_node_copies_no_token_row_and_matches_the_copying_layer(fp8_dispatch):
    from paddleformers_amd import functional as F8
    from paddleformers_amd.fp8_utils import fp8_quant_weight
    from paddleformers_amd.moe_layer import FusionMlpNode
    from tests.test_gpu_fusion_mlp_node import _custom_map, _fresh_experts
    from tests.test_gpu_moe_layer import _layer

    T, H, I, E, topk = 900, 512, 256, 4, 2
    rm, probs, counts, w1, w2, _, x, dy = _layer(T, H, I, E, topk, seed=91)
    trm, tpr = torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
    tokens = F8.fp8_quant_blockwise(G.to_torch_bf16(x), quant_method="1x128") if fp8_dispatch else G.to_torch_bf16(x)
    tdy = G.to_torch_bf16(dy)
    out = []
    for fuse, fwd_rows, bwd_rows in ((False, 0, 0), (True, 0, 0), (False, 256, 256), (True, 256, 256)):
        experts = _fresh_experts(w1, w2)
        fp8_quant_weight([e.w1 for e in experts], [e.w2 for e in experts], batch_mode=True)
        layer = FusionMlpNode(_custom_map(experts, counts), topk, is_split_group_gemm=False, recompute_fwd_gate_up=True,
                              dsv3_use_fp8_dispatch=fp8_dispatch, mlp_fwd_subbatch_rows=fwd_rows if fp8_dispatch else 0,
                              mlp_bwd_subbatch_rows=bwd_rows)
        layer.fuse_unzip = fuse
        y = layer.forward(tokens, trm, tpr)
        assert isinstance(layer.experts_group_gemm_node.input_fp8, F8.GatheredRows) == fuse     # (bf16 tokens: quantized per token first)
        seen = []
        real = layer.experts_group_gemm_node.backward
        layer.experts_group_gemm_node.backward = lambda g, *a, **k: (seen.append(type(g)), real(g, *a, **k))[1]
        dx, dp = layer.backward(tdy)
        assert all((t is F8.GatheredRows) == fuse for t in seen) and seen
        out.append((y, dx, dp, [e.w1.main_grad for e in experts] + [e.w2.main_grad for e in experts]))
    for other in out[1:]:
        assert torch.equal(out[0][0].view(torch.int16), other[0].view(torch.int16))
        assert torch.equal(out[0][1].view(torch.int16), other[1].view(torch.int16)) and torch.equal(out[0][2], other[2])
    # weight gradients: slices accumulate in another order than one pass, so each way of slicing is compared with itself
    for a, b in ((out[0], out[1]), (out[2], out[3])):
        for ga, gb in zip(a[3], b[3]):
            assert (ga is None) == (gb is None) and (ga is None or torch.equal(ga, gb))


def test_row_scales_of_gathered_rows(F):
    T, H, topk, E = 150, 640, 2, 4
    rm, probs, counts = routing(T, topk, E, seed=21)
    q, s = _tokens(T, H, seed=22)
    (cx, _, _, cs), (g, _, _, _) = _both(F, q, s, rm, probs, E, counts)
    rs = g.row_scales()
    assert tuple(rs.shape) == tuple(cs.shape) and rs.stride() == (1, rs.shape[0]) and g.row_scales() is rs      # stored [H/128, rows], made once
    assert torch.equal(rs, cs)                       # zero on padding rows, as the copy writes them
    part = g[128:256]
    assert torch.equal(part.row_scales(), cs[128:256]) and part.row_scales().stride() == (1, 128)
