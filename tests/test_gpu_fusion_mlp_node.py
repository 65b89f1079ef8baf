"""`FusionMlpNode` (cli/train/deepseek_v3_pretrain/moe_layer.py:705-1125): the caller that strings UnZipNode, the FP8 expert
MLP and ZipNode together.  Its parts are pinned elsewhere (permute kernels and the node stage by stage against the oracle);
here the orchestration is checked: same results as the three nodes driven by hand, bf16 and FP8 dispatch, the sub-batched
forward and backward equal to the one-shot passes to the bit, the adaptive recompute switch, and the state it drops."""
import types

import numpy as np
import pytest

from tests import _gen as G
from tests.test_gpu_moe_layer import _Expert, _layer

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _custom_map(experts, counts, seq_length=64, topk=3, ratio=1.0):
    cm = types.SimpleNamespace(tokens_per_expert=list(counts))
    return types.SimpleNamespace(experts=experts, token_dispatcher=types.SimpleNamespace(_comm_manager=cm),
                                 config=types.SimpleNamespace(seq_length=seq_length, num_experts_per_tok=topk,
                                                              adaptive_remained_O1_recompute_ratio=ratio))


def _fresh_experts(w1, w2):
    out = []
    for a, b in zip(w1, w2):
        t1, t2 = G.to_torch_bf16(a), G.to_torch_bf16(b)
        t1.main_grad = None
        t2.main_grad = None
        out.append(_Expert(t1, t2))
    return out


@pytest.mark.parametrize("fp8_dispatch", [False, True])
@pytest.mark.parametrize("split", [True, False])
def test_fusion_mlp_node_equals_the_three_nodes_driven_by_hand(fp8_dispatch, split):
    from paddleformers_amd import functional as F8
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode
    from paddleformers_amd.moe_layer import FusionMlpNode
    from paddleformers_amd.moe_utils import UnZipNode, ZipNode

    T, H, I, E, topk = 300, 512, 256, 6, 3
    rm, probs, counts, w1, w2, _, x, dy = _layer(T, H, I, E, topk, seed=51)
    trm, tpr = torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
    tx, tdy = G.to_torch_bf16(x), G.to_torch_bf16(dy)
    tokens = F8.fp8_quant_blockwise(tx, quant_method="1x128") if fp8_dispatch else tx

    experts = _fresh_experts(w1, w2)
    layer = FusionMlpNode(_custom_map(experts, counts), topk, is_split_group_gemm=split, dsv3_use_fp8_dispatch=fp8_dispatch)
    y = layer.forward(tokens, trm.to(torch.int64), tpr)
    assert layer.padding_token_per_experts == [(c + 127) // 128 * 128 for c in counts] and layer.dispatched_indices.dtype == torch.int32
    dx, dp = layer.backward(tdy)
    assert layer.unzip_node is None and layer.experts_group_gemm_node is None and layer.tokens_per_expert is None    # state dropped

    ref = _fresh_experts(w1, w2)
    padded = [(c + 127) // 128 * 128 for c in counts]
    unzip, zipn = UnZipNode(), ZipNode()
    mlp = FP8GroupGemmMlpFunctionNode(types.SimpleNamespace(experts=ref), is_split_group_gemm=split)
    rows, rowmap, rp, rs = unzip.forward(tokens, trm, tpr, topk, E, counts)
    o3 = mlp.forward((rows, rs) if fp8_dispatch else rows, rp, padded)
    ey = zipn.forward(o3, rowmap, trm, rp, T, E)
    grows = zipn.backward(tdy, trm, tpr, topk, E, counts)
    dxr, pgr = mlp.backward(grows, rp, padded)
    edx, edp = unzip.backward(dxr, T, pgr, trm, E)
    assert torch.equal(y.view(torch.int16), ey.view(torch.int16))
    assert torch.equal(dx.view(torch.int16), edx.view(torch.int16)) and torch.equal(dp, edp)
    for a, b in zip(experts, ref):
        for name in ("w1", "w2"):
            ga, gb = getattr(a, name).main_grad, getattr(b, name).main_grad
            assert (ga is None) == (gb is None) and (ga is None or torch.equal(ga, gb))
    with pytest.raises(ValueError):
        FusionMlpNode(_custom_map(_fresh_experts(w1, w2), counts), topk, dsv3_use_fp8_dispatch=not fp8_dispatch).forward(tokens, trm, tpr)


def test_fusion_mlp_node_subbatches_equal_the_one_shot_passes():
    from paddleformers_amd import functional as F8
    from paddleformers_amd.moe_layer import FusionMlpNode

    T, H, I, E, topk = 700, 512, 256, 4, 2
    rm, probs, counts, w1, w2, _, x, dy = _layer(T, H, I, E, topk, seed=61, drop=0.0)
    trm, tpr = torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
    tokens = F8.fp8_quant_blockwise(G.to_torch_bf16(x), quant_method="1x128")
    grad = F8.fp8_quant_blockwise(G.to_torch_bf16(dy), quant_method="1x128")
    total = sum((c + 127) // 128 * 128 for c in counts)
    assert total > 2 * 256

    def run(fwd_rows, bwd_rows):
        experts = _fresh_experts(w1, w2)
        layer = FusionMlpNode(_custom_map(experts, counts), topk, recompute_fwd_gate_up=True, is_split_group_gemm=False,
                              mlp_fwd_subbatch_rows=fwd_rows, mlp_bwd_subbatch_rows=bwd_rows)
        y = layer.forward(tokens, trm, tpr)
        dx, dp = layer.backward(grad)
        return y, dx, dp, [e.w1.main_grad for e in experts], [e.w2.main_grad for e in experts]

    one = run(0, 0)
    for fwd_rows, bwd_rows in ((256, 0), (0, 256), (256, 256)):
        sub = run(fwd_rows, bwd_rows)
        assert torch.equal(one[0].view(torch.int16), sub[0].view(torch.int16)), (fwd_rows, bwd_rows)
        assert torch.equal(one[1].view(torch.int16), sub[1].view(torch.int16)) and torch.equal(one[2], sub[2])
        # weight gradients accumulate slice by slice: fp32 sums in another order
        for a, b in zip(one[3] + one[4], sub[3] + sub[4]):
            assert (a is None) == (b is None)
            if a is not None:
                assert G.rel_fro(b.cpu().numpy(), a.cpu().numpy()) < 1e-5


def test_fusion_mlp_node_adaptive_recompute_switch():
    from paddleformers_amd.moe_layer import FusionMlpNode

    T, H, I, E, topk = 200, 256, 128, 3, 2
    rm, probs, counts, w1, w2, _, x, _ = _layer(T, H, I, E, topk, seed=71)
    trm, tpr = torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
    total = sum((c + 127) // 128 * 128 for c in counts)
    for ratio, want in ((total / (10.0 * topk) - 1.0, True), (total / (10.0 * topk) + 1.0, False)):
        layer = FusionMlpNode(_custom_map(_fresh_experts(w1, w2), counts, seq_length=10, topk=topk, ratio=ratio), topk,
                              recompute_fwd_gate_up=-1, dsv3_use_fp8_dispatch=False)
        layer.forward(G.to_torch_bf16(x), trm, tpr)
        assert layer.experts_group_gemm_node.recompute_fwd_gate_up is want
        assert (layer.experts_group_gemm_node.o1 is None) == want
