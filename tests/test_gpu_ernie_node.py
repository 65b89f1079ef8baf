"""GPU tests of the masked-layout FP8 expert node (ExpertsGroupGemmNode of the ERNIE token dispatcher)
through its reference-named host mirror: forward stage by stage against the CPU oracle chain, forward and
backward against a plain fp32 MoE at FP8 accuracy, and the switches of fp8_fused_ops_configs."""
import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


class _Lin:
    def __init__(self, w):
        self.weight = w


class _Expert:
    def __init__(self, w1, w2):
        self.up_gate_proj, self.down_proj = _Lin(w1), _Lin(w2)


class _Cfg:
    def __init__(self, d):
        self.fp8_fused_ops_configs = d


class _Map:
    def __init__(self, experts, cfg):
        self.experts, self.config = experts, _Cfg(cfg)


def _make(E, H, I, Mmax, valid, seed):
    """Weights, a masked-layout input whose rows past valid[e] are zero, probs and an output gradient."""
    w1 = [G.bf16_normal((H, 2 * I), seed=seed + e, std=0.03) for e in range(E)]
    w2 = [G.bf16_normal((I, H), seed=seed + 100 + e, std=0.03) for e in range(E)]
    experts = []
    for e in range(E):
        t1, t2 = G.to_torch_bf16(w1[e]), G.to_torch_bf16(w2[e])
        t1.main_grad = None
        t2.main_grad = None
        experts.append(_Expert(t1, t2))
    x = G.bf16_normal((E * Mmax, H), seed=seed + 500).reshape(E, Mmax, H)
    dout = G.bf16_normal((E * Mmax, H), seed=seed + 600, std=1e-3).reshape(E, Mmax, H)
    for e in range(E):
        x[e, valid[e]:] = 0
        dout[e, valid[e]:] = 0
    probs = np.random.default_rng(seed).random(E * Mmax, dtype=np.float32) * 0.5 + 0.25
    return w1, w2, experts, x.reshape(E * Mmax, H), probs, dout


@pytest.mark.parametrize("stack_quant", [True, False])
def test_ernie_node_forward_against_oracle_chain(stack_quant):
    from paddleformers_amd.ernie_fp8_utils import ExpertsGroupGemmNode

    E, H, I, Mmax = 3, 512, 256, 256
    valid = [256, 0, 77]
    w1, w2, experts, x, probs, _ = _make(E, H, I, Mmax, valid, seed=41)
    node = ExpertsGroupGemmNode(experts, _Map(experts, {"stack_quant": stack_quant}))
    tm = torch.tensor(valid, dtype=torch.int32, device="cuda")
    o3 = node.forward(G.to_torch_bf16(x), torch.from_numpy(probs).cuda(), tm)
    assert tuple(o3.shape) == (E, Mmax, H) and o3.dtype == torch.bfloat16
    assert tuple(node.unzipped_probs.shape) == (E, Mmax, 1)
    masked = np.array(valid, np.int32)
    # stage 1: up+gate masked GEMM
    xq, xs = O.quant_1x128(x, 0)
    w1q, w1s = O.stack_transpose_quant(w1, transpose=True)
    eo1 = O.grouped_gemm_nt_masked(xq.reshape(E, Mmax, H), xs.reshape(E, Mmax, H // 128), w1q.reshape(E, 2 * I, H),
                                   w1s.reshape(E, 2 * I // 128, H // 128), masked)
    o1 = G.from_torch_bf16(node.o1)
    for e in range(E):
        v = valid[e]
        if v:
            assert G.rel_fro(O.bf16_bits_to_f32(o1[e, :v]), O.bf16_bits_to_f32(eo1[e, :v])) <= 1e-3
        assert not o1[e, v:].any()          # rows past the valid count keep the zeros of the output buffer
    # stage 2 + 3 from the GPU's own o1: swiglu * probs requantized bit-exactly (plain scales), down GEMM
    q2, s2 = O.swiglu_weighted_quant(o1.reshape(E * Mmax, 2 * I), probs, 0, False)
    w2q, w2s = O.stack_transpose_quant(w2, transpose=True)
    eo3 = O.grouped_gemm_nt_masked(q2.reshape(E, Mmax, I), s2.reshape(E, Mmax, I // 128), w2q.reshape(E, H, I),
                                   w2s.reshape(E, H // 128, I // 128), masked)
    g3 = G.from_torch_bf16(o3)
    for e in range(E):
        v = valid[e]
        if v:
            assert G.rel_fro(O.bf16_bits_to_f32(g3[e, :v]), O.bf16_bits_to_f32(eo3[e, :v])) <= 1e-3
        assert not g3[e, v:].any()


def _fp32_moe(x, probs, w1, w2, E, Mmax, valid, dout, with_probs=True):
    xt = torch.tensor(O.bf16_bits_to_f32(x), dtype=torch.float32, requires_grad=True)
    pt = torch.tensor(probs, dtype=torch.float32, requires_grad=True)
    w1t = [torch.tensor(O.bf16_bits_to_f32(w), requires_grad=True) for w in w1]
    w2t = [torch.tensor(O.bf16_bits_to_f32(w), requires_grad=True) for w in w2]
    out = torch.zeros((E * Mmax, w2[0].shape[1]))
    parts = []
    for e in range(E):
        lo, hi = e * Mmax, e * Mmax + valid[e]
        if hi == lo:
            continue
        h = xt[lo:hi] @ w1t[e]
        I = h.shape[1] // 2
        act = torch.nn.functional.silu(h[:, :I]) * h[:, I:]
        if with_probs:
            act = act * pt[lo:hi, None]
        parts.append((lo, hi, act @ w2t[e]))
    loss = 0.0
    d = torch.tensor(O.bf16_bits_to_f32(dout).reshape(E * Mmax, -1))
    for lo, hi, y in parts:
        out[lo:hi] = y.detach()
        loss = loss + (y * d[lo:hi]).sum()
    loss.backward()
    return (out.numpy(), xt.grad.numpy(), pt.grad.numpy() if with_probs else None, [w.grad for w in w1t], [w.grad for w in w2t])


@pytest.mark.parametrize("cfg", [{"stack_quant": True, "swiglu_probs_bwd": True}, {}])
def test_ernie_node_forward_backward_against_fp32_moe(cfg):
    from paddleformers_amd.ernie_fp8_utils import ExpertsGroupGemmNode

    E, H, I, Mmax = 3, 512, 384, 256
    valid = [256, 130, 0]
    w1, w2, experts, x, probs, dout = _make(E, H, I, Mmax, valid, seed=47)
    node = ExpertsGroupGemmNode(experts, _Map(experts, cfg))
    tm = torch.tensor(valid, dtype=torch.int32, device="cuda")
    o3 = node.forward(G.to_torch_bf16(x), torch.from_numpy(probs).cuda(), tm)
    dx, pg = node.backward(G.to_torch_bf16(dout), tm, None, Mmax)
    assert tuple(dx.shape) == (E * Mmax, H) and tuple(pg.shape) == (E, Mmax)
    assert node.o1 is None and node.unzipped_tokens is None            # backward resets the node
    ref_o3, ref_dx, ref_pg, ref_dw1, ref_dw2 = _fp32_moe(x, probs, w1, w2, E, Mmax, valid, dout)
    assert G.rel_fro(o3.float().cpu().numpy().reshape(E * Mmax, H), ref_o3) < 0.08
    assert G.rel_fro(dx.float().cpu().numpy(), ref_dx) < 0.08
    assert G.rel_fro(pg.cpu().numpy().reshape(-1), ref_pg) < 0.08
    for e in range(E):
        g1, g2 = experts[e].up_gate_proj.weight.main_grad, experts[e].down_proj.weight.main_grad
        assert g1.dtype == torch.float32 and g2.dtype == torch.float32
        if valid[e] == 0:
            assert not g1.any() and not g2.any()
            continue
        assert G.rel_fro(g1.cpu().numpy(), ref_dw1[e].numpy()) < 0.08
        assert G.rel_fro(g2.cpu().numpy(), ref_dw2[e].numpy()) < 0.08
    # a second backward accumulates
    node.forward(G.to_torch_bf16(x), torch.from_numpy(probs).cuda(), tm)
    node.backward(G.to_torch_bf16(dout), tm, None, Mmax)
    g1 = experts[0].up_gate_proj.weight.main_grad
    assert G.rel_fro(g1.cpu().numpy(), 2 * ref_dw1[0].numpy()) < 0.08


@pytest.mark.parametrize("cfg", [{"stack_quant": True, "swiglu_probs_bwd": True}, {}])
def test_ernie_node_backward_with_the_fused_swiglu_backward_is_the_reference_sequence(cfg):
    """The SwiGLU backward that writes do1 and o2_s in quantized form only (row scales [E, Mmax, 2I/128], exact scales in
    both directions) against the reference's calls (fp8_utils.py:371-439, 498-716): dx and the weight gradients to the bit,
    probs_grad to 1e-5 of its largest entry."""
    from paddleformers_amd.ernie_fp8_utils import ExpertsGroupGemmNode

    E, H, I, Mmax = 3, 512, 384, 256
    valid = [256, 130, 0]
    res = []
    for fuse in (False, True):
        w1, w2, experts, x, probs, dout = _make(E, H, I, Mmax, valid, seed=49)
        node = ExpertsGroupGemmNode(experts, _Map(experts, dict(cfg)))
        node.fuse_bwd_quant = fuse
        tm = torch.tensor(valid, dtype=torch.int32, device="cuda")
        node.forward(G.to_torch_bf16(x), torch.from_numpy(probs).cuda(), tm)
        dx, pg = node.backward(G.to_torch_bf16(dout), tm, None, Mmax)
        res.append((dx, pg, [e.up_gate_proj.weight.main_grad for e in experts] + [e.down_proj.weight.main_grad for e in experts]))
    a, b = res
    assert torch.equal(a[0].view(torch.int16), b[0].view(torch.int16))
    for ga, gb in zip(a[2], b[2]):
        assert torch.equal(ga, gb)
    assert tuple(b[1].shape) == (E, Mmax) and float(a[1].abs().max()) > 0
    assert float((a[1] - b[1]).abs().max()) <= 1e-5 * float(a[1].abs().max())


def test_ernie_node_no_prob_path():
    from paddleformers_amd.ernie_fp8_utils import ExpertsGroupGemmNode

    E, H, I, Mmax = 2, 256, 128, 128
    valid = [128, 50]
    w1, w2, experts, x, probs, dout = _make(E, H, I, Mmax, valid, seed=53)
    node = ExpertsGroupGemmNode(experts, _Map(experts, {"stack_quant": True}))
    tm = torch.tensor(valid, dtype=torch.int32, device="cuda")
    o3 = node.forward_no_prob(G.to_torch_bf16(x), tm)
    dx = node.backward_no_prob(G.to_torch_bf16(dout), tm)
    ref_o3, ref_dx, _, ref_dw1, ref_dw2 = _fp32_moe(x, probs, w1, w2, E, Mmax, valid, dout, with_probs=False)
    assert G.rel_fro(o3.float().cpu().numpy().reshape(E * Mmax, H), ref_o3) < 0.08
    assert G.rel_fro(dx.float().cpu().numpy(), ref_dx) < 0.08
    for e in range(E):
        assert G.rel_fro(experts[e].up_gate_proj.weight.main_grad.cpu().numpy(), ref_dw1[e].numpy()) < 0.08
        assert G.rel_fro(experts[e].down_proj.weight.main_grad.cpu().numpy(), ref_dw2[e].numpy()) < 0.08


def test_ernie_node_uses_cached_stacked_weights_and_split_group_gemm():
    from paddleformers_amd import ernie_fp8_utils as EU
    from paddleformers_amd import functional as F8

    E, H, I, Mmax = 2, 256, 128, 128
    w1, w2, experts, x, probs, _ = _make(E, H, I, Mmax, [128, 128], seed=59)
    ws = [ex.up_gate_proj.weight for ex in experts]
    q, s = EU.fused_stack_transpose_quant(ws, transpose=True)
    ws[0].fp8_weight_stacked, ws[0].fp8_scale_stacked = "plain", "plain-scale"
    ws[0].fp8_weight_stacked_transpose, ws[0].fp8_scale_stacked_transpose = q, s
    q2, s2 = EU.fused_stack_transpose_quant(ws, transpose=True)
    assert q2 is q and s2 is s
    assert EU.fused_stack_transpose_quant(ws, transpose=False) == ("plain", "plain-scale")
    assert EU.has_config({"a": 1}, "a") and not EU.has_config({"a": 0}, "a") and not EU.has_config(None, "a")
    # split_group_gemm on a contiguous layout equals the grouped GEMM of the same segments
    xq, xs = F8.fp8_quant_blockwise(G.to_torch_bf16(x), quant_method="1x128", input_transpose=False, output_scale_transpose=False)
    out = torch.zeros((E * Mmax, 2 * I), dtype=torch.bfloat16, device="cuda")
    EU.split_group_gemm(xq, xs, q.reshape(E, 2 * I, H), s.reshape(E, 2 * I // 128, H // 128), [Mmax, Mmax], out)
    from paddleformers_amd import deep_gemm as DG

    ref = torch.zeros_like(out)
    m_idx = torch.arange(E, dtype=torch.int32, device="cuda").repeat_interleave(Mmax)
    DG.m_grouped_fp8_gemm_nt_contiguous((xq, xs), (q.reshape(E, 2 * I, H), s.reshape(E, 2 * I // 128, H // 128)), ref, m_idx)
    assert G.rel_fro(out.float().cpu().numpy(), ref.float().cpu().numpy()) <= 1e-3


def test_ernie_node_rejects_a_ragged_layout():
    from paddleformers_amd.ernie_fp8_utils import ExpertsGroupGemmNode

    E, H, I, Mmax = 3, 256, 128, 128
    w1, w2, experts, x, probs, _ = _make(E, H, I, Mmax, [128] * 3, seed=61)
    node = ExpertsGroupGemmNode(experts, _Map(experts, {}))
    tm = torch.tensor([128] * 3, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        node.forward(G.to_torch_bf16(x[:-128 - 1]), torch.from_numpy(probs).cuda(), tm)


# ---------------------------------------------------------------------------------------------
# ExpertsGroupGemmContiguousNode
# ---------------------------------------------------------------------------------------------

_ALL_FUSED = {"stack_quant": True, "spaq": True, "swiglu_probs_bwd": True, "transpose_split_quant": True}


class _W:
    def __init__(self, w1, w2):
        self.w1, self.w2 = w1, w2


class _TMap:
    def __init__(self, experts):
        self.experts = experts


def _contig_case(E, H, I, rows, seed):
    w1 = [G.bf16_normal((H, 2 * I), seed=seed + e, std=0.03) for e in range(E)]
    w2 = [G.bf16_normal((I, H), seed=seed + 100 + e, std=0.03) for e in range(E)]
    M = sum(rows)
    x = G.bf16_normal((M, H), seed=seed + 500)
    dout = G.bf16_normal((M, H), seed=seed + 600, std=1e-3)
    probs = np.random.default_rng(seed).random(M, dtype=np.float32) * 0.5 + 0.25
    return w1, w2, x, probs, dout


def _ernie_experts(w1, w2):
    ex = []
    for a, b in zip(w1, w2):
        t1, t2 = G.to_torch_bf16(a), G.to_torch_bf16(b)
        t1.main_grad = None
        t2.main_grad = None
        ex.append(_Expert(t1, t2))
    return ex


@pytest.mark.parametrize("fuse_bwd", [True, False])
@pytest.mark.parametrize("dequant_input", [False, True])
@pytest.mark.parametrize("recompute", [False, True])
def test_ernie_contiguous_node_equals_the_transformers_node_when_every_switch_is_on(dequant_input, recompute, fuse_bwd):
    """With stack_quant, spaq, swiglu_probs_bwd and transpose_split_quant the two classes ask for the same
    operators with the same arguments: identical outputs and gradients, with the backward's quantizations fused into
    their producers (both classes' default) and as the reference's sequence of calls."""
    from paddleformers_amd.ernie_fp8_utils import ExpertsGroupGemmContiguousNode
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode

    E, H, I = 3, 512, 384
    rows = [256, 0, 384]
    w1, w2, x, probs, dout = _contig_case(E, H, I, rows, seed=71)
    ex = _ernie_experts(w1, w2)
    node = ExpertsGroupGemmContiguousNode(_Map(ex, dict(_ALL_FUSED)), recompute_fwd_gate_up=recompute, dequant_input=dequant_input)
    node.fuse_bwd_quant = fuse_bwd
    tp = torch.from_numpy(probs).cuda()
    o3 = node.forward(G.to_torch_bf16(x), tp, rows, rows)
    assert tuple(node.unzipped_probs.shape) == (sum(rows), 1)
    dx, pg = node.backward(G.to_torch_bf16(dout))
    assert node.o1 is None and node.m_indices is None           # backward resets the node

    tex = []
    for a, b in zip(w1, w2):
        t1, t2 = G.to_torch_bf16(a), G.to_torch_bf16(b)
        t1.main_grad = None
        t2.main_grad = None
        tex.append(_W(t1, t2))
    ref = FP8GroupGemmMlpFunctionNode(_TMap(tex), recompute_fwd_gate_up=recompute)
    ref.fuse_bwd_quant = ref.fuse_bwd_swiglu_quant = fuse_bwd
    r3 = ref.forward(G.to_torch_bf16(x), tp.unsqueeze(-1), rows)
    rdx, rpg = ref.backward(G.to_torch_bf16(dout), tp.unsqueeze(-1), rows)
    assert torch.equal(o3, r3) and torch.equal(dx, rdx) and torch.equal(pg, rpg)
    for e in range(E):
        if rows[e] == 0:
            continue
        assert torch.equal(ex[e].down_proj.weight.main_grad, tex[e].w2.main_grad)
        g1, r1 = ex[e].up_gate_proj.weight.main_grad, tex[e].w1.main_grad
        if dequant_input:
            assert torch.equal(g1, r1)      # both transpose the dequantized FP8 copy of the input
        else:
            assert G.rel_fro(g1.cpu().numpy(), r1.cpu().numpy()) < 0.06     # this one transposes the bf16 input itself


@pytest.mark.parametrize("cfg", [{}, {"split_group_gemm": True}, {"stack_quant": True, "transpose_split_quant": True}])
def test_ernie_contiguous_node_against_fp32_moe(cfg):
    from paddleformers_amd.ernie_fp8_utils import ExpertsGroupGemmContiguousNode

    E, H, I = 3, 512, 256
    rows = [128, 256, 0]
    w1, w2, x, probs, dout = _contig_case(E, H, I, rows, seed=83)
    ex = _ernie_experts(w1, w2)
    node = ExpertsGroupGemmContiguousNode(_Map(ex, dict(cfg)))
    tp = torch.from_numpy(probs).cuda()
    o3 = node.forward(G.to_torch_bf16(x), tp, rows, rows)
    calls = []

    class _Task:
        def wait(self):
            calls.append("wait")

    def a2a(t):
        calls.append("start")
        return t, _Task()

    dx, pg = node.backward(G.to_torch_bf16(dout), a2a_async_fn=a2a)
    assert calls == ["start", "wait"]
    # the masked-layout helper of this file, with every expert's capacity equal to its segment, is the same MoE
    off, refs = 0, []
    for e, r in enumerate(rows):
        refs.append((off, r))
        off += r
    xt = torch.tensor(O.bf16_bits_to_f32(x), requires_grad=True)
    pt = torch.tensor(probs, requires_grad=True)
    w1t = [torch.tensor(O.bf16_bits_to_f32(w), requires_grad=True) for w in w1]
    w2t = [torch.tensor(O.bf16_bits_to_f32(w), requires_grad=True) for w in w2]
    d = torch.tensor(O.bf16_bits_to_f32(dout))
    outs = torch.zeros((sum(rows), H))
    loss = 0.0
    for e, (lo, r) in enumerate(refs):
        if r == 0:
            continue
        h = xt[lo:lo + r] @ w1t[e]
        y = (torch.nn.functional.silu(h[:, :I]) * h[:, I:] * pt[lo:lo + r, None]) @ w2t[e]
        outs[lo:lo + r] = y.detach()
        loss = loss + (y * d[lo:lo + r]).sum()
    loss.backward()
    assert G.rel_fro(o3.float().cpu().numpy(), outs.numpy()) < 0.08
    assert G.rel_fro(dx.float().cpu().numpy(), xt.grad.numpy()) < 0.08
    assert G.rel_fro(pg.cpu().numpy(), pt.grad.numpy()) < 0.08
    for e, (lo, r) in enumerate(refs):
        if r:
            assert G.rel_fro(ex[e].up_gate_proj.weight.main_grad.cpu().numpy(), w1t[e].grad.numpy()) < 0.08
            assert G.rel_fro(ex[e].down_proj.weight.main_grad.cpu().numpy(), w2t[e].grad.numpy()) < 0.08


@pytest.mark.parametrize("cfg", [{}, dict(_ALL_FUSED)])
@pytest.mark.parametrize("dequant_input", [False, True])
def test_ernie_contiguous_node_backward_with_fused_quantizations_is_the_reference_sequence(cfg, dequant_input):
    """One read of out_grad for its two quantizations and a SwiGLU backward that writes quantized forms only, against the
    reference's sequence of calls (fp8_utils.py:1345-1436): dx and the weight gradients to the bit, probs_grad (summed in
    another order) to 1e-5 of its largest entry."""
    from paddleformers_amd.ernie_fp8_utils import ExpertsGroupGemmContiguousNode

    E, H, I = 3, 512, 384
    rows = [256, 0, 384]
    w1, w2, x, probs, dout = _contig_case(E, H, I, rows, seed=91)
    tp = torch.from_numpy(probs).cuda()
    res = []
    for fuse in (False, True):
        ex = _ernie_experts(w1, w2)
        node = ExpertsGroupGemmContiguousNode(_Map(ex, dict(cfg)), dequant_input=dequant_input)
        node.fuse_bwd_quant = fuse
        node.forward(G.to_torch_bf16(x), tp, rows, rows)
        dx, pg = node.backward(G.to_torch_bf16(dout))
        res.append((dx, pg, [e.up_gate_proj.weight.main_grad for e in ex], [e.down_proj.weight.main_grad for e in ex]))
    a, b = res
    assert torch.equal(a[0].view(torch.int16), b[0].view(torch.int16))
    for ga, gb in zip(a[2] + a[3], b[2] + b[3]):
        assert (ga is None) == (gb is None) and (ga is None or torch.equal(ga, gb))
    assert float(a[1].abs().max()) > 0 and float((a[1] - b[1]).abs().max()) <= 1e-5 * float(a[1].abs().max())


def test_ernie_contiguous_node_zero_rows_and_prequantized_input():
    from paddleformers_amd import functional as F8
    from paddleformers_amd.ernie_fp8_utils import ExpertsGroupGemmContiguousNode

    E, H, I = 2, 256, 128
    rows = [128, 128]
    w1, w2, x, probs, dout = _contig_case(E, H, I, rows, seed=89)
    ex = _ernie_experts(w1, w2)
    node = ExpertsGroupGemmContiguousNode(_Map(ex, dict(_ALL_FUSED)))
    o = node.forward(torch.zeros((0, H), dtype=torch.bfloat16, device="cuda"), torch.zeros((0,), device="cuda"), [0, 0], [0, 0])
    assert tuple(o.shape) == (0, H)
    dx, pg = node.backward(torch.zeros((0, H), dtype=torch.bfloat16, device="cuda"))
    assert tuple(dx.shape) == (0, H) and tuple(pg.shape) == (0, 1)
    assert all(e.up_gate_proj.weight.main_grad is not None and not e.up_gate_proj.weight.main_grad.any() for e in ex)
    # an (fp8, scale) input needs dequant_input
    xq, xs = F8.fp8_quant_blockwise(G.to_torch_bf16(x), quant_method="1x128", input_transpose=False, output_scale_transpose=False)
    tp = torch.from_numpy(probs).cuda()
    with pytest.raises(AssertionError):
        node.forward(xq, tp, rows, rows, scale=xs)
    node2 = ExpertsGroupGemmContiguousNode(_Map(ex, dict(_ALL_FUSED)), dequant_input=True)
    a = node2.forward(xq, tp, rows, rows, scale=xs)
    node3 = ExpertsGroupGemmContiguousNode(_Map(ex, dict(_ALL_FUSED)))
    b = node3.forward(G.to_torch_bf16(x), tp, rows, rows)
    assert torch.equal(a, b)
