"""Tokens in, tokens out: UnZipNode -> FP8GroupGemmMlpFunctionNode -> ZipNode, forward and backward, as the reference's
MoE layer chains them (cli/train/deepseek_v3_pretrain/moe_utils.py:130-261 around transformers/fp8_utils.py:913-1321).

Every stage is pinned against the oracle elsewhere (permute kernels bit-exact, the node stage by stage); here the chain
is compared with a plain fp32 autograd MoE on the same bf16 values at FP8 accuracy, and the two nodes' own contracts
(padding rows, the row map handed from one to the other, FP8 tokens with scales) are checked exactly.
"""
import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


class _Expert:
    def __init__(self, w1, w2):
        self.w1, self.w2 = w1, w2


class _Map:
    def __init__(self, experts):
        self.experts = experts


def _layer(T, H, I, E, topk, seed, drop=0.1):
    rng = np.random.default_rng(seed)
    rm = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    rm[rng.random(rm.shape) < drop] = -1
    rm[:, 1][rm[:, 1] == 1] = -1
    rm[rm == 1] = -1                                            # expert 1 receives nothing
    counts = [int((rm == e).sum()) for e in range(E)]
    probs = (rng.random(rm.shape) * 0.5 + 0.25).astype(np.float32)
    w1 = [G.bf16_normal((H, 2 * I), seed=seed + e, std=0.03) for e in range(E)]
    w2 = [G.bf16_normal((I, H), seed=seed + 100 + e, std=0.03) for e in range(E)]
    experts = []
    for e in range(E):
        t1, t2 = G.to_torch_bf16(w1[e]), G.to_torch_bf16(w2[e])
        t1.main_grad = None
        t2.main_grad = None
        experts.append(_Expert(t1, t2))
    x = G.bf16_normal((T, H), seed=seed + 500)
    dy = G.bf16_normal((T, H), seed=seed + 600, std=1e-3)
    return rm, probs, counts, w1, w2, experts, x, dy


def _fp32_layer(x, rm, probs, w1, w2, dy):
    """y[t] = sum over the token's used slots of probs[t, k] * MLP_e(x[t]), fp32 autograd."""
    xt = torch.tensor(O.bf16_bits_to_f32(x), requires_grad=True)
    pt = torch.tensor(probs, requires_grad=True)
    w1t = [torch.tensor(O.bf16_bits_to_f32(w), requires_grad=True) for w in w1]
    w2t = [torch.tensor(O.bf16_bits_to_f32(w), requires_grad=True) for w in w2]
    y = torch.zeros_like(xt)
    for e in range(len(w1)):
        t_idx, k_idx = np.nonzero(rm == e)
        if len(t_idx) == 0:
            continue
        h = xt[t_idx] @ w1t[e]
        I = h.shape[1] // 2
        act = torch.nn.functional.silu(h[:, :I]) * h[:, I:] * pt[t_idx, k_idx][:, None]
        y = y.index_add(0, torch.tensor(t_idx), act @ w2t[e])
    y.backward(torch.tensor(O.bf16_bits_to_f32(dy)))
    return y.detach().numpy(), xt.grad.numpy(), pt.grad.numpy(), [w.grad for w in w1t], [w.grad for w in w2t]


@pytest.mark.parametrize("fp8_tokens", [False, True])
def test_tokens_through_unzip_node_experts_zip_node_and_back(fp8_tokens):
    from paddleformers_amd import functional as F8
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode
    from paddleformers_amd.moe_utils import UnZipNode, ZipNode

    T, H, I, E, topk = 300, 512, 256, 6, 3
    rm, probs, counts, w1, w2, experts, x, dy = _layer(T, H, I, E, topk, seed=11)
    padded = [(c + 127) // 128 * 128 for c in counts]
    assert counts[1] == 0 and min(c for i, c in enumerate(counts) if i != 1) > 0
    trm, tpr = torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
    tx, tdy = G.to_torch_bf16(x), G.to_torch_bf16(dy)
    unzip, zipn, mlp = UnZipNode(), ZipNode(), FP8GroupGemmMlpFunctionNode(_Map(experts))

    # ---- forward
    tokens = F8.fp8_quant_blockwise(tx, quant_method="1x128") if fp8_tokens else tx      # FP8 dispatch hands (bytes, scales)
    rows, rowmap, row_probs, row_scale = unzip.forward(tokens, trm, tpr, topk, E, counts)
    assert rows.shape[0] == sum(padded) and rowmap.shape == (T, E) and row_probs.shape == (sum(padded), 1)
    assert (row_scale is not None) == fp8_tokens
    start = 0
    for e in range(E):                                          # padding rows: zero bytes, zero probability
        pad = slice(start + counts[e], start + padded[e])
        assert not rows[pad].view(torch.uint8).any() and not row_probs[pad].any()
        start += padded[e]
    o3 = mlp.forward((rows, row_scale) if fp8_tokens else rows, row_probs, padded)
    y = zipn.forward(o3, rowmap, trm, row_probs, T, E)
    assert y.shape == (T, H) and y.dtype == torch.bfloat16

    # ---- backward
    grad_rows = zipn.backward(tdy, trm, tpr, topk, E, counts)
    assert grad_rows.shape == o3.shape
    dx_rows, probs_grad_rows = mlp.backward(grad_rows, row_probs, padded)
    dx, dprobs = unzip.backward(dx_rows, T, probs_grad_rows, trm, E)
    assert unzip.zipped_expertwise_rowmap is None               # the node drops its state after backward
    assert dx.shape == (T, H) and dprobs.shape == (T, topk)

    # the two reordering passes that carry numbers, pinned to the bit against the oracle on the very rows they were
    # handed (fp32 sum of a token's copies in slot order, bf16 out), independently of the FP8 noise of the MLP between them
    ey, _ = O.moe_unpermute(G.from_torch_bf16(o3), rowmap.cpu().numpy(), rm, row_probs.cpu().numpy(), T, E)
    assert (G.from_torch_bf16(y) == ey).all(), "ZipNode.forward differs from the oracle's moe_unpermute"
    edx, edp = O.moe_unpermute(G.from_torch_bf16(dx_rows), rowmap.cpu().numpy(), rm, probs_grad_rows.cpu().numpy(), T, E)
    assert (G.from_torch_bf16(dx) == edx).all(), "UnZipNode.backward differs from the oracle's moe_unpermute"
    assert (dprobs.cpu().numpy() == edp).all(), "UnZipNode.backward: probability gradients differ from the oracle's"

    ref_y, ref_dx, ref_dp, ref_dw1, ref_dw2 = _fp32_layer(x, rm, probs, w1, w2, dy)
    errs = {"y": G.rel_fro(y.float().cpu().numpy(), ref_y), "dx": G.rel_fro(dx.float().cpu().numpy(), ref_dx)}
    print("layer errors vs fp32:", errs)
    # measured on MI355X: 0.065 for y and for dx (the e4m3 rounding of two GEMM operands in a row; inputs, weights and
    # routing all come from the seeds above).  The bar is 1.4 times that: a dropped probability factor, a wrong expert or
    # a missing copy in the sum moves these errors to 0.3 and beyond.
    tol = 0.09
    assert G.rel_fro(y.float().cpu().numpy(), ref_y) < tol
    assert G.rel_fro(dx.float().cpu().numpy(), ref_dx) < tol
    used = rm >= 0
    assert G.rel_fro(dprobs.cpu().numpy()[used], ref_dp[used]) < tol
    assert not dprobs.cpu().numpy()[~used].any()                # unused slots get no gradient
    for e in range(E):
        if counts[e]:
            assert G.rel_fro(experts[e].w1.main_grad.cpu().numpy(), ref_dw1[e].numpy()) < tol
            assert G.rel_fro(experts[e].w2.main_grad.cpu().numpy(), ref_dw2[e].numpy()) < tol


def test_zip_node_backward_takes_fp8_gradients_with_scales():
    from paddleformers_amd import functional as F8
    from paddleformers_amd.moe_utils import UnZipNode, ZipNode

    T, H, E, topk = 200, 384, 5, 2
    rm, probs, counts, *_ , x, dy = _layer(T, H, 128, E, topk, seed=23)
    trm, tpr = torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
    q, s = F8.fp8_quant_blockwise(G.to_torch_bf16(dy), quant_method="1x128")
    rows, scale = ZipNode().backward((q, s), trm, tpr, topk, E, counts)
    eq, erow, _, es = O.moe_permute(G.from_torch_fp8(q), s.cpu().numpy(), rm, probs, E, counts, 128)
    assert (G.from_torch_fp8(rows) == eq).all() and (scale.cpu().numpy() == es).all()
    # the same reordering as UnZipNode.forward on the same routing
    rows2, rowmap, _, scale2 = UnZipNode().forward((q, s), trm, tpr, topk, E, counts)
    assert torch.equal(rows.view(torch.uint8), rows2.view(torch.uint8)) and torch.equal(scale, scale2)
    assert (rowmap.cpu().numpy() == erow).all()
    with pytest.raises(ValueError):
        UnZipNode().forward(G.to_torch_bf16(x), trm, tpr, topk + 1, E, counts)
    with pytest.raises(RuntimeError):
        UnZipNode().backward(rows, T, None, trm, E)


def test_reordering_nodes_issue_no_host_synchronisation():
    """The reference's moe_permute / moe_unpermute calls return without a device-to-host round trip
    (moe_utils.py:157-181, 205-212); torch's synchronisation debug mode turns any `.item()` / blocking copy into an
    error, so the four node passes must get through it."""
    from paddleformers_amd import functional as F8
    from paddleformers_amd.moe_utils import UnZipNode, ZipNode

    T, H, E, topk = 200, 384, 5, 2
    rm, probs, counts, *_, x, dy = _layer(T, H, 128, E, topk, seed=31)
    trm, tpr = torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda()
    xt, dyt = G.to_torch_bf16(x), G.to_torch_bf16(dy)
    unzip, zipn = UnZipNode(), ZipNode()
    F8.moe_permute_check()                       # allocates the flag word of this device, outside the guarded region
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("error")
    try:
        rows, rowmap, up, _ = unzip.forward(xt, trm, tpr, topk, E, counts)
        y = zipn.forward(rows, rowmap, trm, up, T, E)
        drows = zipn.backward(dyt, trm, tpr, topk, E, counts)
        dx, dp = unzip.backward(drows, T, up, trm, E)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    torch.cuda.synchronize()
    F8.moe_permute_check()                       # consistent counts: nothing flagged
    assert y.shape == (T, H) and dx.shape == (T, H) and dp.shape == (T, topk)
