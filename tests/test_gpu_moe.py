"""GPU tests of the fused FP8 MoE node (forward and backward) through the reference-named host
mirror: against the CPU oracle chain stage by stage, and against a plain fp32 MoE at FP8 accuracy."""
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


def _make(E, H, I, rows, seed):
    w1 = [G.bf16_normal((H, 2 * I), seed=seed + e, std=0.03) for e in range(E)]
    w2 = [G.bf16_normal((I, H), seed=seed + 100 + e, std=0.03) for e in range(E)]
    experts = []
    for e in range(E):
        t1, t2 = G.to_torch_bf16(w1[e]), G.to_torch_bf16(w2[e])
        t1.main_grad = None
        t2.main_grad = None
        experts.append(_Expert(t1, t2))
    M = sum(rows)
    x = G.bf16_normal((M, H), seed=seed + 500)
    probs = np.random.default_rng(seed).random(M, dtype=np.float32) * 0.5 + 0.25
    return w1, w2, experts, x, probs


def _oracle_forward(x, probs, w1, w2, rows):
    E = len(rows)
    H, I2 = w1[0].shape
    I = I2 // 2
    m_idx = np.repeat(np.arange(E, dtype=np.int32), rows)
    xq, xs = O.quant_1x128(x, 0)
    w1q, w1s = O.stack_transpose_quant(w1, transpose=True)
    w2q, w2s = O.stack_transpose_quant(w2, transpose=True)
    o1 = O.grouped_gemm_nt_contiguous(xq, xs, w1q.reshape(E, I2, H), w1s.reshape(E, I2 // 128, H // 128), m_idx)
    return o1, m_idx, (w2q.reshape(E, H, I), w2s.reshape(E, H // 128, I // 128))


@pytest.mark.parametrize("split", [False, True])
def test_moe_node_forward_against_oracle_chain(split):
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode

    E, H, I = 4, 512, 256
    rows = [128, 0, 256, 128]
    w1, w2, experts, x, probs = _make(E, H, I, rows, seed=1)
    node = FP8GroupGemmMlpFunctionNode(_Map(experts), is_split_group_gemm=split)
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    o3 = node.forward(G.to_torch_bf16(x), tp, rows)
    assert tuple(o3.shape) == (sum(rows), H) and o3.dtype == torch.bfloat16
    # stage 1: up+gate GEMM vs oracle
    eo1, m_idx, (w2q, w2s) = _oracle_forward(x, probs, w1, w2, rows)
    o1 = G.from_torch_bf16(node.o1)
    assert G.rel_fro(O.bf16_bits_to_f32(o1), O.bf16_bits_to_f32(eo1)) <= 1e-3
    # stage 2+3 from the GPU's own o1: requant bit-exact (pow2 scales, as the node asks), then down GEMM
    q2, s2 = O.swiglu_weighted_quant(o1, probs, 0, True)
    eo3 = O.grouped_gemm_nt_contiguous(q2, s2, w2q, w2s, m_idx)
    assert G.rel_fro(O.bf16_bits_to_f32(G.from_torch_bf16(o3)), O.bf16_bits_to_f32(eo3)) <= 1e-3
    # cached quantised input is what a re-run with hs_out=None consumes
    o3b = node.forward(None, tp, rows)
    assert torch.equal(o3.view(torch.int16), o3b.view(torch.int16))
    # (fp8, scale) tuple input gives the same result
    from paddleformers_amd import functional as F8

    xq, xs = F8.fp8_quant_blockwise(G.to_torch_bf16(x), quant_method="1x128", output_scale_transpose=False)
    node2 = FP8GroupGemmMlpFunctionNode(_Map(experts), is_split_group_gemm=split)
    o3c = node2.forward((xq, xs), tp, rows)
    assert torch.equal(o3.view(torch.int16), o3c.view(torch.int16))


def test_moe_node_zero_rows_and_recompute():
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode

    E, H, I = 2, 256, 128
    w1, w2, experts, x, probs = _make(E, H, I, [128, 128], seed=3)
    node = FP8GroupGemmMlpFunctionNode(_Map(experts), recompute_fwd_gate_up=True)
    out = node.forward(torch.zeros((0, H), dtype=torch.bfloat16, device="cuda"), torch.zeros((0, 1), device="cuda"), [0, 0])
    assert tuple(out.shape) == (0, H)
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    o3 = node.forward(G.to_torch_bf16(x), tp, [128, 128])
    assert node.o1 is None       # recompute mode does not keep o1
    dx, pg = node.backward(torch.randn((256, H), device="cuda").to(torch.bfloat16) * 1e-3, tp, [128, 128])
    assert tuple(dx.shape) == (256, H) and tuple(pg.shape) == (256,)


def _fp32_moe(x, probs, w1, w2, rows, dout):
    """Plain fp32 autograd MoE on the bf16 values: the semantics of nn/experts.py:50-69 with the
    probs multiply of the fused node."""
    xt = torch.tensor(O.bf16_bits_to_f32(x), dtype=torch.float32, requires_grad=True)
    pt = torch.tensor(probs, dtype=torch.float32, requires_grad=True)
    w1t = [torch.tensor(O.bf16_bits_to_f32(w), requires_grad=True) for w in w1]
    w2t = [torch.tensor(O.bf16_bits_to_f32(w), requires_grad=True) for w in w2]
    outs, off = [], 0
    for e, r in enumerate(rows):
        if r == 0:
            continue
        h = xt[off:off + r] @ w1t[e]
        I = h.shape[1] // 2
        act = torch.nn.functional.silu(h[:, :I]) * h[:, I:] * pt[off:off + r, None]
        outs.append(act @ w2t[e])
        off += r
    out = torch.cat(outs)
    out.backward(torch.tensor(O.bf16_bits_to_f32(dout)))
    return out.detach().numpy(), xt.grad.numpy(), pt.grad.numpy(), [w.grad for w in w1t], [w.grad for w in w2t]


def test_moe_node_forward_backward_against_fp32_moe():
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode

    E, H, I = 3, 512, 256
    rows = [256, 0, 128]
    w1, w2, experts, x, probs = _make(E, H, I, rows, seed=7)
    dout = G.bf16_normal((sum(rows), H), seed=9, std=1e-3)
    node = FP8GroupGemmMlpFunctionNode(_Map(experts))
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    o3 = node.forward(G.to_torch_bf16(x), tp, rows)
    dx, pg = node.backward(G.to_torch_bf16(dout), tp, rows)
    ref_o3, ref_dx, ref_pg, ref_dw1, ref_dw2 = _fp32_moe(x, probs, w1, w2, rows, dout)
    # FP8 quantisation noise: a few percent relative Frobenius at these sizes
    assert G.rel_fro(o3.float().cpu().numpy(), ref_o3) < 0.08
    assert G.rel_fro(dx.float().cpu().numpy(), ref_dx) < 0.08
    assert G.rel_fro(pg.cpu().numpy(), ref_pg) < 0.08
    for e, r in enumerate(rows):
        if r == 0:
            assert experts[e].w1.main_grad is None and experts[e].w2.main_grad is None
            continue
        assert G.rel_fro(experts[e].w1.main_grad.cpu().numpy(), ref_dw1[e].numpy()) < 0.08
        assert G.rel_fro(experts[e].w2.main_grad.cpu().numpy(), ref_dw2[e].numpy()) < 0.08
    # a second backward accumulates into main_grad
    g1 = experts[0].w1.main_grad.clone()
    node.forward(G.to_torch_bf16(x), tp, rows)
    node.backward(G.to_torch_bf16(dout), tp, rows)
    assert torch.allclose(experts[0].w1.main_grad, 2 * g1, rtol=1e-5, atol=1e-8)


def test_moe_backward_stages_against_oracle():
    """dgrad-down -> SwiGLU backward -> dgrad-up, each stage fed with the GPU's previous stage and
    compared with the oracle; weight gradients compared with the oracle's wgrad GEMM."""
    from paddleformers_amd import functional as F8
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode

    E, H, I = 2, 256, 128
    rows = [128, 256]
    w1, w2, experts, x, probs = _make(E, H, I, rows, seed=11)
    dout = G.bf16_normal((sum(rows), H), seed=12, std=1e-3)
    node = FP8GroupGemmMlpFunctionNode(_Map(experts))
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    node.forward(G.to_torch_bf16(x), tp, rows)
    o1 = node.o1
    expert_w1 = [e.w1 for e in experts]
    expert_w2 = [e.w2 for e in experts]
    do1, o2_s, pg = node.bwd_dowm_input(expert_w2, G.to_torch_bf16(dout), o1, rows, unzipped_probs=tp)
    m_idx = np.repeat(np.arange(E, dtype=np.int32), rows)
    dq, ds = O.quant_1x128(dout, 0)
    w2q, w2s = O.stack_transpose_quant(w2, transpose=False)         # [E*I, H]: NT operand of dgrad-down
    edo2 = O.grouped_gemm_nt_contiguous(dq, ds, w2q.reshape(E, I, H), w2s.reshape(E, I // 128, H // 128), m_idx)
    edo1, epg, eo2s = O.swiglu_weighted_bwd(G.from_torch_bf16(o1), edo2, probs)
    assert np.array_equal(G.from_torch_bf16(o2_s), eo2s)
    assert G.rel_fro(O.bf16_bits_to_f32(G.from_torch_bf16(do1)), O.bf16_bits_to_f32(edo1)) <= 5e-3
    dx = node.bwd_gate_up_input(do1, expert_w1, rows)
    d1q, d1s = O.quant_1x128(G.from_torch_bf16(do1), 0)
    w1q, w1s = O.stack_transpose_quant(w1, transpose=False)          # [E*H, 2I]
    edx = O.grouped_gemm_nt_contiguous(d1q, d1s, w1q.reshape(E, H, 2 * I), w1s.reshape(E, H // 128, 2 * I // 128), m_idx)
    assert G.rel_fro(O.bf16_bits_to_f32(G.from_torch_bf16(dx)), O.bf16_bits_to_f32(edx)) <= 1e-3
    # weight gradient of w2 for expert 1 from the GPU's transposed operands vs the oracle GEMM
    a_t, sa_t = F8.fused_transpose_split_quant(o2_s, None, rows, True)
    b_t, sb_t = F8.fused_transpose_split_quant(G.to_torch_bf16(dout), None, rows, True)
    node.bwd_down_weight((b_t, sb_t), (a_t, sa_t), expert_w2, rows)
    e = 1
    exp = O.gemm_nt_1d1d_f32(G.from_torch_fp8(a_t[e]), sa_t[e].cpu().numpy(), G.from_torch_fp8(b_t[e]), sb_t[e].cpu().numpy())
    assert G.rel_fro(experts[e].w2.main_grad.cpu().numpy(), exp) <= 5e-5


def test_moe_backward_grouped_wgrad_when_main_grads_are_stacked():
    """Experts whose main_grad tensors are slices of one buffer get their weight gradients from one
    grouped launch; the result equals the per-expert loop."""
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode

    E, H, I = 4, 512, 256
    rows = [256, 0, 128, 384]
    w1, w2, experts, x, probs = _make(E, H, I, rows, seed=21)
    dout = G.bf16_normal((sum(rows), H), seed=22, std=1e-3)
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    # reference: separate main_grad tensors (allocated on first use), per-expert loop
    node = FP8GroupGemmMlpFunctionNode(_Map(experts))
    node.forward(G.to_torch_bf16(x), tp, rows)
    dx_ref, pg_ref = node.backward(G.to_torch_bf16(dout), tp, rows)
    ref1 = [e.w1.main_grad for e in experts]
    ref2 = [e.w2.main_grad for e in experts]
    # stacked buffers
    g1 = torch.zeros((E, H, 2 * I), dtype=torch.float32, device="cuda")
    g2 = torch.zeros((E, I, H), dtype=torch.float32, device="cuda")
    for e in range(E):
        experts[e].w1.main_grad, experts[e].w2.main_grad = g1[e], g2[e]
    assert FP8GroupGemmMlpFunctionNode._stacked_main_grad([e.w1 for e in experts]) is not None
    node.forward(G.to_torch_bf16(x), tp, rows)
    dx, pg = node.backward(G.to_torch_bf16(dout), tp, rows)
    assert torch.equal(dx, dx_ref) and torch.equal(pg, pg_ref)
    for e in range(E):
        if rows[e] == 0:
            assert ref1[e] is None and not g1[e].any() and not g2[e].any()
        else:
            assert torch.equal(g1[e], ref1[e]) and torch.equal(g2[e], ref2[e])
    # not stacked: one expert's gradient lives elsewhere
    experts[2].w1.main_grad = torch.zeros((H, 2 * I), dtype=torch.float32, device="cuda")
    assert FP8GroupGemmMlpFunctionNode._stacked_main_grad([e.w1 for e in experts]) is None


# ---------------------------------------------------------------------------------------------
# use_ue8m0: power-of-two scales everywhere, forward-type GEMMs on the block-scaled MFMA kernel
# ---------------------------------------------------------------------------------------------


def test_moe_node_ue8m0_forward_against_oracle_chain():
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode

    E, H, I = 4, 512, 384
    rows = [128, 0, 384, 256]
    w1, w2, experts, x, probs = _make(E, H, I, rows, seed=21)
    node = FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=True)
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    o3 = node.forward(G.to_torch_bf16(x), tp, rows)
    m_idx = np.repeat(np.arange(E, dtype=np.int32), rows)
    xq, xs = O.quant_1x128(x, 0, pow2=True)
    w1q, w1s = O.stack_transpose_quant(w1, transpose=True, pow2=True)
    w2q, w2s = O.stack_transpose_quant(w2, transpose=True, pow2=True)
    eo1 = O.grouped_gemm_nt_contiguous(xq, xs, w1q.reshape(E, 2 * I, H), w1s.reshape(E, 2 * I // 128, H // 128), m_idx)
    o1 = G.from_torch_bf16(node.o1)
    assert G.rel_fro(O.bf16_bits_to_f32(o1), O.bf16_bits_to_f32(eo1)) <= 1e-3
    q2, s2 = O.swiglu_weighted_quant(o1, probs, 0, True)
    eo3 = O.grouped_gemm_nt_contiguous(q2, s2, w2q.reshape(E, H, I), w2s.reshape(E, H // 128, I // 128), m_idx)
    assert G.rel_fro(O.bf16_bits_to_f32(G.from_torch_bf16(o3)), O.bf16_bits_to_f32(eo3)) <= 1e-3
    assert node._group_items is not None      # one work-item list served both GEMMs


def test_moe_node_ue8m0_forward_backward_against_fp32_moe():
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode

    E, H, I = 3, 512, 384
    rows = [256, 0, 384]
    w1, w2, experts, x, probs = _make(E, H, I, rows, seed=27)
    dout = G.bf16_normal((sum(rows), H), seed=29, std=1e-3)
    node = FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=True)
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    o3 = node.forward(G.to_torch_bf16(x), tp, rows)
    dx, pg = node.backward(G.to_torch_bf16(dout), tp, rows)
    ref_o3, ref_dx, ref_pg, ref_dw1, ref_dw2 = _fp32_moe(x, probs, w1, w2, rows, dout)
    # power-of-two scales cost up to one bit of the FP8 mantissa: a little above the 0.08 of the exact scales
    assert G.rel_fro(o3.float().cpu().numpy(), ref_o3) < 0.10
    assert G.rel_fro(dx.float().cpu().numpy(), ref_dx) < 0.10
    assert G.rel_fro(pg.cpu().numpy(), ref_pg) < 0.10
    for e, r in enumerate(rows):
        if r:
            assert G.rel_fro(experts[e].w1.main_grad.cpu().numpy(), ref_dw1[e].numpy()) < 0.10
            assert G.rel_fro(experts[e].w2.main_grad.cpu().numpy(), ref_dw2[e].numpy()) < 0.10


def test_moe_node_ue8m0_needs_a_pow2_weight_cache():
    from paddleformers_amd import fp8_utils as U

    E, H, I = 2, 512, 384
    rows = [256, 256]
    _, _, experts, x, probs = _make(E, H, I, rows, seed=31)
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    plain = U.FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=True).forward(G.to_torch_bf16(x), tp, rows)
    U.fp8_quant_weight([e.w1 for e in experts], [e.w2 for e in experts], batch_mode=True)
    with pytest.raises(RuntimeError):
        U.FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=True).forward(G.to_torch_bf16(x), tp, rows)
    for e in experts:
        for w in (e.w1, e.w2):
            for name in ("fp8_weight_stacked", "fp8_scale_stacked", "fp8_weight_stacked_transpose", "fp8_scale_stacked_transpose",
                         "fp8_scale_is_pow2"):
                if hasattr(w, name):
                    delattr(w, name)
    U.fp8_quant_weight([e.w1 for e in experts], [e.w2 for e in experts], batch_mode=True, using_pow2_scale=True)
    cached = U.FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=True).forward(G.to_torch_bf16(x), tp, rows)
    assert torch.equal(plain.view(torch.int16), cached.view(torch.int16))


def test_moe_node_ue8m0_iteration_runs_no_scale_conversion_pass(monkeypatch):
    """With the weight cache warm, a use_ue8m0 iteration converts no scale tensor: every activation quantizer writes the
    exponent bytes itself.  Results equal those of the fp32-scale quantizers followed by the conversion, to the bit."""
    from paddleformers_amd import fp8_utils as U
    from paddleformers_amd import functional as F8

    E, H, I = 3, 512, 384
    rows = [256, 0, 384]
    _, _, experts, x, probs = _make(E, H, I, rows, seed=43)
    dout = G.bf16_normal((sum(rows), H), seed=44, std=1e-3)
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    tx, tdo = G.to_torch_bf16(x), G.to_torch_bf16(dout)
    U.fp8_quant_weight([e.w1 for e in experts], [e.w2 for e in experts], batch_mode=True, using_pow2_scale=True)
    converted = []
    real = F8.scales_to_ue8m0

    def counting(scale, check=True):
        if scale.dtype == torch.float32:
            converted.append(tuple(scale.shape))
        return real(scale, check)

    monkeypatch.setattr(F8, "scales_to_ue8m0", counting)

    def run(node):
        for e in experts:
            e.w1.main_grad = None
            e.w2.main_grad = None
        o3 = node.forward(tx, tp, rows).clone()
        dx, pg = node.backward(tdo, tp, rows)
        return o3, dx.clone(), pg.clone(), [e.w1.main_grad.clone() for e in experts if e.w1.main_grad is not None]

    run(U.FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=True))           # warm: the weights' bytes are made here
    converted.clear()
    node = U.FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=True)
    got = run(node)
    assert converted == [] and node._scale_bytes
    # the expert-by-expert loop takes fp32 scales; it is the same arithmetic
    loop = U.FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=True, is_split_group_gemm=True)
    assert not loop._scale_bytes
    ref = run(loop)
    assert torch.equal(got[0].view(torch.int16), ref[0].view(torch.int16)) and torch.equal(got[1].view(torch.int16), ref[1].view(torch.int16))
    # probs_grad: the loop's SwiGLU backward sums a row in one pass, the grouped node's per column tile
    assert float((got[2] - ref[2]).abs().max()) <= 1e-5 * float(ref[2].abs().max())
    for a, b in zip(got[3], ref[3]):
        assert G.rel_fro(a.cpu().numpy(), b.cpu().numpy()) < 1e-6


def test_moe_node_ue8m0_weight_scale_bytes_follow_the_weight_cache():
    """The node remembers the UE8M0 bytes of the cached weight scales between calls; a new cache (new tensors) and a
    cache rewritten in place (same tensors, new contents) must both be picked up."""
    from paddleformers_amd import fp8_utils as U
    from paddleformers_amd import functional as F8

    E, H, I = 2, 512, 384
    rows = [256, 384]
    _, _, experts, x, probs = _make(E, H, I, rows, seed=37)
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    tx = G.to_torch_bf16(x)
    names = ("fp8_weight_stacked", "fp8_scale_stacked", "fp8_weight_stacked_transpose", "fp8_scale_stacked_transpose", "fp8_scale_is_pow2")

    def recache():
        for e in experts:
            for w in (e.w1, e.w2):
                for name in names:
                    if hasattr(w, name):
                        delattr(w, name)
        U.fp8_quant_weight([e.w1 for e in experts], [e.w2 for e in experts], batch_mode=True, using_pow2_scale=True)

    recache()
    node = U.FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=True)
    first = node.forward(tx, tp, rows).clone()
    again = node.forward(tx, tp, rows)
    assert torch.equal(first.view(torch.int16), again.view(torch.int16))
    # the bytes of the w1 and w2 scales are kept next to the cache they were made from, converted once
    kept = experts[0].w1.fp8_scale_stacked_transpose_ue8m0
    assert kept[0] is experts[0].w1.fp8_scale_stacked_transpose and experts[0].w2.fp8_scale_stacked_transpose_ue8m0[2].dtype == torch.uint8
    node.forward(tx, tp, rows)
    assert experts[0].w1.fp8_scale_stacked_transpose_ue8m0 is kept
    # new weights, new cache
    with torch.no_grad():
        for e in experts:
            e.w1.mul_(4.0)
            e.w2.mul_(0.5)
    recache()
    fresh = U.FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=True).forward(tx, tp, rows)
    same_node = node.forward(tx, tp, rows)
    assert torch.equal(fresh.view(torch.int16), same_node.view(torch.int16))
    assert not torch.equal(first.view(torch.int16), same_node.view(torch.int16))
    # the cache rewritten in place
    with torch.no_grad():
        for e in experts:
            e.w1.mul_(0.25)
    w0 = experts[0].w1
    q, s = F8.fused_stack_transpose_quant([e.w1 for e in experts], transpose=True, using_pow2_scale=True)
    w0.fp8_weight_stacked_transpose.copy_(q)
    w0.fp8_scale_stacked_transpose.copy_(s)
    q, s = F8.fused_stack_transpose_quant([e.w1 for e in experts], transpose=False, using_pow2_scale=True)
    w0.fp8_weight_stacked.copy_(q)
    w0.fp8_scale_stacked.copy_(s)
    fresh = U.FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=True).forward(tx, tp, rows)
    same_node = node.forward(tx, tp, rows)
    assert torch.equal(fresh.view(torch.int16), same_node.view(torch.int16))


@pytest.mark.parametrize("ue8m0", [False, True])
def test_moe_node_backward_fused_gradient_quantization_is_bit_identical(ue8m0):
    # backward quantizes out_grad and do1 once (row-wise + transposed from one read) or twice (the
    # reference's call sequence): same dx, probs_grad and weight gradients to the bit
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode

    E, H, I = 3, 512, 384
    rows = [256, 0, 384]
    w1, w2, experts, x, probs = _make(E, H, I, rows, seed=31)
    dout = G.to_torch_bf16(G.bf16_normal((sum(rows), H), seed=33, std=1e-3))
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    # ... or not at all for do1 and o2_s, which the SwiGLU backward then writes in their quantized forms only: same dx and
    # weight gradients to the bit, probs_grad (a sum taken in another order) to 1e-5 of the magnitudes of its terms
    res = []
    for fuse, fuse_act in ((True, False), (False, False), (True, True)):
        for ex in experts:
            ex.w1.main_grad = torch.zeros_like(ex.w1, dtype=torch.float32)
            ex.w2.main_grad = torch.zeros_like(ex.w2, dtype=torch.float32)
        node = FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=ue8m0)
        node.fuse_bwd_quant, node.fuse_bwd_swiglu_quant = fuse, fuse_act
        node.forward(G.to_torch_bf16(x), tp, rows)
        dx, pg = node.backward(dout, tp, rows)
        res.append((dx, pg, [ex.w1.main_grad for ex in experts], [ex.w2.main_grad for ex in experts]))
    a, b, c = res
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]) and torch.equal(a[0], c[0])
    for ga, gb, gc in zip(a[2] + a[3], b[2] + b[3], c[2] + c[3]):
        assert torch.equal(ga, gb) and torch.equal(ga, gc)
    assert float(a[1].abs().max()) > 0
    assert float((a[1] - c[1]).abs().max()) <= 1e-5 * float(a[1].abs().max()) + 1e-30


# ---------------------------------------------------------------------------------------------
# sub-batched forward / backward and deferred weight gradients
# ---------------------------------------------------------------------------------------------


def _split_list_prefix(counts, start, end):
    """Rows of every expert that fall into [start, end): what the caller hands to a sub-batch
    (cli/train/deepseek_v3_pretrain/moe_layer.py:838-851)."""
    out, off = [], 0
    for c in counts:
        out.append(max(0, min(end, off + c) - max(start, off)))
        off += c
    return out


@pytest.mark.parametrize("ue8m0", [False, True])
def test_moe_node_subbatches_equal_the_one_shot_node(ue8m0):
    """The caller's sub-batch loops (moe_layer.py:791-884, 936-982, 1054-1103): the quantised input is cut
    into slices of a multiple of 128 rows that straddle experts, each slice goes through forward / backward
    with its own m_indices slice.  Outputs, dx and probs_grad equal the one-shot node bit for bit; the fp32
    weight gradients are sums split differently, so they agree to rounding."""
    from paddleformers_amd import functional as F8
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode

    E, H, I = 4, 512, 384
    rows = [384, 0, 256, 640]
    M = sum(rows)
    w1, w2, experts, x, probs = _make(E, H, I, rows, seed=41)
    dout = G.to_torch_bf16(G.bf16_normal((M, H), seed=43, std=1e-3))
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    xq, xs = F8.fp8_quant_blockwise(G.to_torch_bf16(x), quant_method="1x128", output_scale_transpose=False, using_pow2_scale=ue8m0)

    def fresh_grads():
        for ex in experts:
            ex.w1.main_grad = torch.zeros_like(ex.w1, dtype=torch.float32)
            ex.w2.main_grad = torch.zeros_like(ex.w2, dtype=torch.float32)

    # one shot
    fresh_grads()
    node = FP8GroupGemmMlpFunctionNode(_Map(experts), recompute_fwd_gate_up=True, use_ue8m0=ue8m0)
    o3_ref = node.forward((xq, xs), tp, rows)
    dx_ref, pg_ref = node.backward(dout, tp, rows)
    g_ref = [(ex.w1.main_grad.clone(), ex.w2.main_grad.clone()) for ex in experts]

    # sub-batched: 512-row slices (the last one 256), cutting through experts 0, 2 and 3
    fresh_grads()
    node = FP8GroupGemmMlpFunctionNode(_Map(experts), recompute_fwd_gate_up=True, use_ue8m0=ue8m0)
    m_indices = node.gen_m_indices(rows)
    node.input_fp8, node.input_scale = xq, xs          # prepare_env_subbatch, moe_layer.py:774-780
    node.fwd_subbatch = True
    step = 512
    parts = [(s, min(s + step, M)) for s in range(0, M, step)]
    outs = [node.forward((xq[s:e], xs[s:e]), tp[s:e], rows, m_indices=m_indices[s:e]) for s, e in parts]
    assert torch.equal(torch.cat(outs).view(torch.int16), o3_ref.view(torch.int16))
    node.bwd_subbatch = True
    dxs, pgs = [], []
    for i, (s, e) in enumerate(parts):
        dx, pg = node.backward(dout[s:e].contiguous(), tp[s:e].contiguous(), _split_list_prefix(rows, s, e),
                               input_fp8_slice=xq[s:e].contiguous(), input_scale_slice=xs[s:e].contiguous(),
                               m_indices=m_indices[s:e].contiguous(), reset_status=i == len(parts) - 1)
        dxs.append(dx)
        pgs.append(pg)
    assert torch.equal(torch.cat(dxs).view(torch.int16), dx_ref.view(torch.int16))
    assert torch.equal(torch.cat(pgs), pg_ref)
    assert node.input_fp8 is None and node.m_indices is None        # the last part released the saved state
    for ex, (r1, r2) in zip(experts, g_ref):
        assert G.rel_fro(ex.w1.main_grad.cpu().numpy(), r1.cpu().numpy()) <= 5e-5 or not r1.any()
        assert G.rel_fro(ex.w2.main_grad.cpu().numpy(), r2.cpu().numpy()) <= 5e-5 or not r2.any()
        assert ex.w1.main_grad.any() == r1.any()


@pytest.mark.parametrize("stacked", [False, True])
def test_moe_node_deferred_weight_gradients_run_at_flush_on_another_stream(stacked):
    """WeightGradStore.enabled (zero-bubble pipeline, fp8_utils.py:314-327): backward queues the weight-gradient
    closures and returns; flush() runs them later, here on a second stream after the activations the node
    held have been dropped.  main_grad ends up bit-identical to the immediate run."""
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode, WeightGradStore

    E, H, I = 3, 512, 256
    rows = [256, 0, 384]
    w1, w2, experts, x, probs = _make(E, H, I, rows, seed=51)
    dout = G.to_torch_bf16(G.bf16_normal((sum(rows), H), seed=53, std=1e-3))
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)

    def fresh_grads():
        if stacked:
            g1 = torch.zeros((E, H, 2 * I), dtype=torch.float32, device="cuda")
            g2 = torch.zeros((E, I, H), dtype=torch.float32, device="cuda")
            for e, ex in enumerate(experts):
                ex.w1.main_grad, ex.w2.main_grad = g1[e], g2[e]
        else:
            for ex in experts:
                ex.w1.main_grad = torch.zeros_like(ex.w1, dtype=torch.float32)
                ex.w2.main_grad = torch.zeros_like(ex.w2, dtype=torch.float32)

    fresh_grads()
    node = FP8GroupGemmMlpFunctionNode(_Map(experts))
    node.forward(G.to_torch_bf16(x), tp, rows)
    dx_ref, pg_ref = node.backward(dout, tp, rows)
    ref = [(ex.w1.main_grad.clone(), ex.w2.main_grad.clone()) for ex in experts]

    fresh_grads()
    node = FP8GroupGemmMlpFunctionNode(_Map(experts))
    node.forward(G.to_torch_bf16(x), tp, rows)
    WeightGradStore.clear()
    WeightGradStore.enabled = True
    try:
        dx, pg = node.backward(dout, tp, rows, reset_status=True)
    finally:
        WeightGradStore.enabled = False
    assert torch.equal(dx, dx_ref) and torch.equal(pg, pg_ref)
    for ex in experts:
        assert not ex.w1.main_grad.any() and not ex.w2.main_grad.any()      # nothing has run yet
    assert len(WeightGradStore._queue) == 2
    # unrelated work reuses the allocator's freed blocks before the closures run
    junk = [torch.randn((sum(rows), H), device="cuda") for _ in range(8)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        WeightGradStore.flush()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    del junk
    assert not WeightGradStore._queue
    for e, (ex, (r1, r2)) in enumerate(zip(experts, ref)):
        assert torch.equal(ex.w1.main_grad, r1) and torch.equal(ex.w2.main_grad, r2), f"expert {e}"
        assert bool(r1.any()) == (rows[e] > 0)


def test_moe_node_reads_fragment_major_copies_of_the_cached_weights():
    """With the per-step FP8 weight cache in place the node's forward-type grouped GEMMs read a fragment-major copy of
    every cached weight whose shape the kernel takes, made once and kept next to the cache entry; the results are those of
    the plain-weight kernels, and a replaced cache entry is picked up."""
    from paddleformers_amd import fp8_utils as U

    E, H, I = 3, 512, 384                    # 2I = 768 and H = 512 are whole 256-column tiles; I = 384 ends in a half tile (dgrad-down)
    rows = [256, 0, 384]
    _, _, experts, x, probs = _make(E, H, I, rows, seed=41)
    dout = G.bf16_normal((sum(rows), H), seed=42, std=1e-3)
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    tx, tdo = G.to_torch_bf16(x), G.to_torch_bf16(dout)
    U.fp8_quant_weight([e.w1 for e in experts], [e.w2 for e in experts], batch_mode=True, fragment_major=False)

    def run(fragment_major):
        for e in experts:
            e.w1.main_grad = None
            e.w2.main_grad = None
        node = U.FP8GroupGemmMlpFunctionNode(_Map(experts))
        node.use_fragment_major = fragment_major
        o3 = node.forward(tx, tp, rows).clone()
        dx, pg = node.backward(tdo, tp, rows)
        return o3, dx.clone(), pg.clone()

    plain = run(False)
    w0, v0 = experts[0].w1, experts[0].w2
    assert not hasattr(w0, "fp8_weight_stacked_transpose_fragment_major")
    fm = run(True)
    for a, b in zip(plain, fm):
        assert torch.equal(a.view(torch.int16) if a.dtype == torch.bfloat16 else a, b.view(torch.int16) if b.dtype == torch.bfloat16 else b)
    kept = w0.fp8_weight_stacked_transpose_fragment_major
    assert kept[0] is w0.fp8_weight_stacked_transpose and isinstance(kept[2], U.deep_gemm.FragmentMajor)
    assert hasattr(v0, "fp8_weight_stacked_transpose_fragment_major") and hasattr(w0, "fp8_weight_stacked_fragment_major")
    assert hasattr(v0, "fp8_weight_stacked_fragment_major")              # [E, I, H] with I = 384: a whole tile and a half one
    run(True)
    assert w0.fp8_weight_stacked_transpose_fragment_major is kept        # made once
    # a new cache entry (next optimizer step) is another tensor: its copy replaces the old one
    with torch.no_grad():
        for e in experts:
            e.w1.mul_(2.0)
    for name in ("fp8_weight_stacked", "fp8_scale_stacked", "fp8_weight_stacked_transpose", "fp8_scale_stacked_transpose"):
        delattr(w0, name)
    U.fp8_quant_weight([e.w1 for e in experts], [e.w2 for e in experts], batch_mode=True, fragment_major=False)
    fresh_plain, fresh_fm = run(False), run(True)
    assert torch.equal(fresh_plain[0].view(torch.int16), fresh_fm[0].view(torch.int16))
    assert not torch.equal(fresh_fm[0].view(torch.int16), fm[0].view(torch.int16))
    assert w0.fp8_weight_stacked_transpose_fragment_major is not kept


@pytest.mark.parametrize("all_layers", [False, True])
def test_weight_requantization_writes_the_fragment_major_copies_the_node_reads(monkeypatch, all_layers):
    """fp8_quant_weight (the per-optimizer-step caller, modeling.py:506-567) makes the fragment-major copies in the pass that
    quantizes the weights: the node's GEMMs then run no re-ordering pass, the copies are the bytes that pass would have
    written, and the results are those of a cache without them."""
    from paddleformers_amd import deep_gemm as dg
    from paddleformers_amd import fp8_utils as U

    E, H, I = 3, 512, 384
    rows = [256, 0, 384]
    _, _, experts, x, probs = _make(E, H, I, rows, seed=47)
    dout = G.bf16_normal((sum(rows), H), seed=48, std=1e-3)
    tp = torch.from_numpy(probs).cuda().unsqueeze(-1)
    tx, tdo = G.to_torch_bf16(x), G.to_torch_bf16(dout)
    names = ("fp8_weight_stacked", "fp8_scale_stacked", "fp8_weight_stacked_transpose", "fp8_scale_stacked_transpose")

    def quantize(**kw):
        for w in (experts[0].w1, experts[0].w2):
            for name in names + tuple(n + "_fragment_major" for n in names):
                if hasattr(w, name):
                    delattr(w, name)
        if all_layers:
            U.fp8_quant_weight_all_layers([([e.w1 for e in experts], [e.w2 for e in experts])], **kw)
        else:
            U.fp8_quant_weight([e.w1 for e in experts], [e.w2 for e in experts], batch_mode=True, **kw)

    def run():
        for e in experts:
            e.w1.main_grad = None
            e.w2.main_grad = None
        node = U.FP8GroupGemmMlpFunctionNode(_Map(experts))
        o3 = node.forward(tx, tp, rows).clone()
        dx, pg = node.backward(tdo, tp, rows)
        return o3, dx.clone(), pg.clone()

    quantize(fragment_major=False)
    lazy = run()
    made_lazily = {n: getattr(experts[0].w1, n + "_fragment_major")[2].data.clone() for n in ("fp8_weight_stacked", "fp8_weight_stacked_transpose")}
    quantize()                                        # default: fp32 scales -> the copies come with the cache
    calls = []
    real = dg.to_fragment_major
    monkeypatch.setattr(dg, "to_fragment_major", lambda w: calls.append(tuple(w.shape)) or real(w))
    w0, v0 = experts[0].w1, experts[0].w2
    for w in (w0, v0):
        for n in ("fp8_weight_stacked", "fp8_weight_stacked_transpose"):
            slot = getattr(w, n + "_fragment_major")
            assert slot[0] is getattr(w, n) and isinstance(slot[2], dg.FragmentMajor)
            assert torch.equal(slot[2].data.view(torch.uint8), real(getattr(w, n).view(slot[2].shape)).data.view(torch.uint8))
    for n, t in made_lazily.items():
        assert torch.equal(getattr(w0, n + "_fragment_major")[2].data.view(torch.uint8), t.view(torch.uint8))
    eager = run()
    assert calls == []
    for a, b in zip(lazy, eager):
        assert torch.equal(a.view(torch.int16) if a.dtype == torch.bfloat16 else a, b.view(torch.int16) if b.dtype == torch.bfloat16 else b)
    # power-of-two scales (use_ue8m0): the node's GEMMs read the plain bytes, no copy is made unless asked for
    quantize(using_pow2_scale=True)
    assert not hasattr(w0, "fp8_weight_stacked_fragment_major")
    quantize(using_pow2_scale=True, fragment_major=True)
    assert hasattr(w0, "fp8_weight_stacked_fragment_major")
