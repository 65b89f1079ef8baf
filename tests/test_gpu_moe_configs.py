"""BASELINE configs 3 and 5 at their own size through FP8GroupGemmMlpFunctionNode.

Every kernel-level call the node makes (quantizers, grouped GEMMs, SwiGLU forward/backward, grouped
weight gradients) is recorded with its inputs and outputs while the node runs once; afterwards each
recorded launch is checked
  * at full size against an fp32 dequantize-then-matmul on the GPU (GEMMs, weight gradients), and
  * on 128-row slabs against the CPU oracle (bit-exact for bytes, scales and elementwise bf16 results;
    the stated Frobenius bars for GEMMs): the largest expert's first and last tile, a one-tile expert
    and the tile that follows an empty expert.
Tolerances are those of tests/test_gpu_gemm.py: 1e-3 relative Frobenius against
bf16(dequant(a) @ dequant(b)^T), 6e-4 against the block-accumulating oracle, fp32 weight gradients
1e-4 (the running sum stays inside the matrix pipe when the scales are powers of two).
"""
import contextlib

import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

REL_FRO = 1e-3
BLOCK_FRO = 6e-4
F32_FRO_MFMA_ACC = 1e-4


class _Expert:
    def __init__(self, w1, w2):
        self.w1, self.w2 = w1, w2


class _Map:
    def __init__(self, experts):
        self.experts = experts


class _Recorder:
    """Patches the operator mirrors the node calls so that every call is kept as (name, args, kwargs, result)."""

    F8_NAMES = ["fp8_quant_blockwise", "fused_weighted_swiglu_act_quant", "fused_transpose_split_quant",
                "quant_and_transpose_split", "fused_swiglu_weighted_bwd", "swiglu_weighted_bwd_quant", "grouped_wgrad"]

    def __init__(self):
        self.calls = []

    def __enter__(self):
        from paddleformers_amd import deep_gemm
        from paddleformers_amd import functional as F8

        self._stack = contextlib.ExitStack()
        for mod, names in ((F8, self.F8_NAMES), (deep_gemm, ["m_grouped_fp8_gemm_nt_contiguous", "m_grouped_fp8_gemm_nt_contiguous_swiglu_quant"])):
            for name in names:
                orig = getattr(mod, name)

                def wrapper(*args, _orig=orig, _name=name, **kwargs):
                    res = _orig(*args, **kwargs)
                    self.calls.append((_name, args, kwargs, res))
                    return res

                setattr(mod, name, wrapper)
                self._stack.callback(setattr, mod, name, orig)
        return self

    def __exit__(self, *exc):
        self._stack.close()
        return False

    def named(self, name):
        return [c for c in self.calls if c[0] == name]


def _scales_f32(s):
    """Scale tensor as the GEMM received it (fp32, or UE8M0 exponent bytes) -> fp32 values, same shape."""
    if s.dtype == torch.float32:
        return s
    return torch.exp2(s.view(torch.uint8).to(torch.float32) - 127.0)


def _slab_tiles(rows):
    """128-row slabs to check against the oracle: (first row, expert, label)."""
    rows = [int(r) for r in rows]
    off = np.concatenate([[0], np.cumsum(rows)]).astype(np.int64)
    big = int(np.argmax(rows))
    picks = [(int(off[big]), big, "largest expert, first tile"), (int(off[big + 1]) - 128, big, "largest expert, last tile")]
    one = [e for e, r in enumerate(rows) if r == 128]
    if one:
        picks.append((int(off[one[0]]), one[0], "one-tile expert"))
    after = [e for e in range(1, len(rows)) if rows[e - 1] == 0 and rows[e] > 0]
    if after:
        picks.append((int(off[after[0]]), after[0], "first tile after an empty expert"))
    return picks


def _check_grouped_gemm(call, rows, what):
    """One recorded m_grouped_fp8_gemm_nt_contiguous: full size on the GPU, slabs against the oracle."""
    _, args, kwargs, _ = call
    (a, sa), (b, sb), out, m_idx = args[0], args[1], args[2], args[3]
    sa, sb = _scales_f32(sa), _scales_f32(sb)
    E, N, K = b.shape
    assert tuple(sa.shape) == (a.shape[0], K // 128) and tuple(sb.shape) == (E, N // 128, K // 128), what
    assert torch.equal(m_idx.cpu(), torch.repeat_interleave(torch.arange(E, dtype=torch.int32), torch.tensor(rows)))
    num = den = 0.0
    off = 0
    for e, r in enumerate(rows):
        if r == 0:
            continue
        ad = a[off:off + r].float() * sa[off:off + r].repeat_interleave(128, dim=1)
        wd = b[e].float() * sb[e].repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
        ref = (ad @ wd.t()).to(torch.bfloat16).float()
        num += float((out[off:off + r].float() - ref).pow(2).sum())
        den += float(ref.pow(2).sum())
        off += r
    err = (num / max(den, 1e-300)) ** 0.5
    assert err <= REL_FRO, f"{what}: full-size rel-Frobenius vs fp32 dequant-matmul {err:.3e}"
    for lo, e, label in _slab_tiles(rows):
        an, san = G.from_torch_fp8(a[lo:lo + 128]), sa[lo:lo + 128].contiguous().cpu().numpy()
        bn, sbn = G.from_torch_fp8(b[e]), sb[e].contiguous().cpu().numpy()
        got = O.bf16_bits_to_f32(G.from_torch_bf16(out[lo:lo + 128]))
        e_ref = G.rel_fro(got, O.bf16_bits_to_f32(O.gemm_nt(an, san, bn, sbn, dequant_ref=True)))
        e_blk = G.rel_fro(got, O.bf16_bits_to_f32(O.gemm_nt(an, san, bn, sbn)))
        assert e_ref <= REL_FRO, f"{what}, {label}: vs oracle dequant-matmul {e_ref:.3e}"
        assert e_blk <= BLOCK_FRO, f"{what}, {label}: vs block-accumulating oracle {e_blk:.3e}"


def _check_quant_rows(x, q, s_kmajor, rows, pow2, what):
    """Row-wise 1x128 quantization of bf16 x (scales stored [K/128, M], fp32 or the UE8M0 bytes the quantizer wrote in
    that mode) on the slabs, bit-exact."""
    s_kmajor = _scales_f32(s_kmajor)
    for lo, _, label in _slab_tiles(rows):
        eq, es = O.quant_1x128(G.from_torch_bf16(x[lo:lo + 128]), 0, pow2=pow2)
        msg = G.mismatch_report(G.from_torch_fp8(q[lo:lo + 128]), eq, f"{what}, {label}: bytes")
        assert not msg, msg
        msg = G.mismatch_report(s_kmajor[:, lo:lo + 128].t().contiguous().cpu().numpy(), es, f"{what}, {label}: scales")
        assert not msg, msg


def _check_transposed(x_slices, q_t, s_t, rows, experts, what):
    """Per-expert transposed quantization (power-of-two scales) of the listed experts, bit-exact.
    x_slices(e) returns the oracle's input for expert e: bf16 bits, or (e4m3 bytes, fp32 scales [M_e, K/128])."""
    for e in experts:
        src = x_slices(e)
        if isinstance(src, tuple):
            eq, es = O.transpose_split_quant(src[0], src[1], [rows[e]], pow2=True)
        else:
            eq, es = O.transpose_split_quant(src, None, [rows[e]], pow2=True)
        msg = G.mismatch_report(G.from_torch_fp8(q_t[e]), eq[0], f"{what}, expert {e}: transposed bytes")
        assert not msg, msg
        msg = G.mismatch_report(s_t[e].cpu().numpy(), es[0], f"{what}, expert {e}: transposed scales")
        assert not msg, msg


def _check_grouped_wgrad(call, rows, what):
    """One recorded grouped_wgrad (into zeroed gradients): every expert against an fp32 dequant-matmul on
    the GPU, the smallest expert and a 256-row slab of the largest against the oracle's wgrad GEMM."""
    _, args, kwargs, _ = call
    a_t, sa_t, b_t, sb_t, out = args[:5]
    for e, r in enumerate(rows):
        if r == 0:
            assert not out[e].any(), f"{what}: expert {e} has no rows but a gradient"
            continue
        A = a_t[e].float() * sa_t[e].repeat_interleave(128, dim=0).t()
        B = b_t[e].float() * sb_t[e].repeat_interleave(128, dim=0).t()
        ref = A @ B.t()
        err = float((out[e] - ref).norm() / ref.norm().clamp_min(1e-30))
        assert err <= F32_FRO_MFMA_ACC, f"{what}: expert {e} ({r} rows) rel-Frobenius vs fp32 dequant-matmul {err:.3e}"
    nz = [e for e, r in enumerate(rows) if r > 0]
    small, big = min(nz, key=lambda e: rows[e]), max(nz, key=lambda e: rows[e])
    for e, sl, label in ((small, slice(None), "smallest expert"), (big, slice(0, 256), "largest expert, rows 0..255")):
        exp = O.gemm_nt_1d1d_f32(G.from_torch_fp8(a_t[e][sl]), sa_t[e][:, sl].contiguous().cpu().numpy(),
                                 G.from_torch_fp8(b_t[e]), sb_t[e].cpu().numpy())
        err = G.rel_fro(out[e][sl].cpu().numpy(), exp)
        assert err <= F32_FRO_MFMA_ACC, f"{what}, {label}: vs oracle {err:.3e}"


def _build(E, H, I, routed, zipf_s, seed, n_empty, ue8m0=False):
    from paddleformers_amd.fp8_utils import FP8GroupGemmMlpFunctionNode

    counts, padded = G.zipf_counts(routed, E, zipf_s, seed=seed, n_empty=n_empty)
    rows = [int(r) for r in padded]
    Mpad = sum(rows)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    g1 = torch.zeros((E, H, 2 * I), dtype=torch.float32, device="cuda")
    g2 = torch.zeros((E, I, H), dtype=torch.float32, device="cuda")
    experts = []
    for e in range(E):
        w1 = (torch.randn((H, 2 * I), generator=gen, device="cuda") * 0.02).to(torch.bfloat16)
        w2 = (torch.randn((I, H), generator=gen, device="cuda") * 0.02).to(torch.bfloat16)
        w1.main_grad, w2.main_grad = g1[e], g2[e]
        experts.append(_Expert(w1, w2))
    # routed rows N(0,1), padding rows zero (what moe_permute hands over)
    x = torch.zeros((Mpad, H), dtype=torch.bfloat16, device="cuda")
    probs = torch.zeros((Mpad, 1), dtype=torch.float32, device="cuda")
    off = 0
    for e in range(E):
        c = int(counts[e])
        if c:
            x[off:off + c] = torch.randn((c, H), generator=gen, device="cuda").to(torch.bfloat16)
            probs[off:off + c, 0] = torch.rand((c,), generator=gen, device="cuda") * 0.5 + 0.25
        off += rows[e]
    node = FP8GroupGemmMlpFunctionNode(_Map(experts), use_ue8m0=ue8m0)
    return node, experts, x, probs, rows, counts, (g1, g2)


def _check_forward(rec, node, x, probs, rows, pow2_in, tag):
    """Checks every launch of one recorded forward; returns o1."""
    qx = rec.named("fp8_quant_blockwise")
    gemms = rec.named("m_grouped_fp8_gemm_nt_contiguous")
    sw = rec.named("fused_weighted_swiglu_act_quant")
    fused = rec.named("m_grouped_fp8_gemm_nt_contiguous_swiglu_quant")
    xq, xs = qx[0][3]
    _check_quant_rows(x, xq, xs, rows, pow2_in, f"{tag} quant(X)")
    if fused:
        # one launch for up+gate GEMM, SwiGLU and requantization: its o1 output is checked like the GEMM's own
        assert len(qx) == 1 and len(gemms) == 1 and not sw, [c[0] for c in rec.calls]
        _, fargs, fkw, (o2q, o2s) = fused[0]
        o1 = fkw["out"]
        assert o1 is not None and fkw["using_pow2_scaling"] is True
        _check_grouped_gemm(("gemm", (fargs[0], fargs[1], o1, fargs[2]), {}, None), rows, f"{tag} up+gate (fused launch)")
        gemms = [None, gemms[0]]
    else:
        assert len(qx) == 1 and len(gemms) == 2 and len(sw) == 1, [c[0] for c in rec.calls]
        _check_grouped_gemm(gemms[0], rows, f"{tag} up+gate")
        o1 = sw[0][1][0]
        o2q, o2s = sw[0][3]
    # SwiGLU + requant (power-of-two scales) of the GPU's own o1, bit-exact on the slabs
    for lo, _, label in _slab_tiles(rows):
        eq, es = O.swiglu_weighted_quant(G.from_torch_bf16(o1[lo:lo + 128]), probs[lo:lo + 128, 0].cpu().numpy(), 0, True)
        msg = G.mismatch_report(G.from_torch_fp8(o2q[lo:lo + 128]), eq, f"{tag} o2 bytes, {label}")
        assert not msg, msg
        msg = G.mismatch_report(_scales_f32(o2s)[lo:lo + 128].contiguous().cpu().numpy(), es, f"{tag} o2 scales, {label}")
        assert not msg, msg
    _check_grouped_gemm(gemms[1], rows, f"{tag} down")
    return o1


@pytest.mark.parametrize("fused", [True, False])
def test_config3_forward_at_full_size(fused):
    """32 experts, hidden 7168, intermediate 2048, 8192 routed rows, Zipf(1.1), two empty experts (the
    benchmark's workload): quant -> up+gate -> SwiGLU+requant -> down, with the middle two as one launch
    (the node's default) and as two."""
    torch.backends.cuda.matmul.allow_tf32 = False
    node, experts, x, probs, rows, counts, _ = _build(32, 7168, 2048, 8192, 1.1, seed=3, n_empty=2)
    node.fuse_swiglu_epilogue = fused
    assert (counts == 0).sum() >= 2 and sum(rows) == 9984
    with _Recorder() as rec:
        o3 = node.forward(x, probs, rows)
    assert tuple(o3.shape) == (sum(rows), 7168)
    assert bool(rec.named("m_grouped_fp8_gemm_nt_contiguous_swiglu_quant")) == fused
    _check_forward(rec, node, x, probs, rows, False, "config 3" + (" fused" if fused else ""))
    if fused:
        # the one-launch forward is the two-launch forward, bit for bit, with and without o1 being kept
        o1_fused = node.o1
        node.fuse_swiglu_epilogue = False
        o3_two = node.forward(None, probs, rows)
        assert torch.equal(o3.view(torch.int16), o3_two.view(torch.int16))
        assert torch.equal(o1_fused.view(torch.int16), node.o1.view(torch.int16))
        node.fuse_swiglu_epilogue, node.recompute_fwd_gate_up = True, True
        node.o1 = None
        o3_no_o1 = node.forward(None, probs, rows)
        assert node.o1 is None and torch.equal(o3.view(torch.int16), o3_no_o1.view(torch.int16))
    # rows of padding stay exactly zero through the whole pipeline (zero input rows, zero probabilities)
    off = 0
    for e, r in enumerate(rows):
        c = int(counts[e])
        assert not o3[off + c:off + r].any()
        off += r


@pytest.mark.parametrize("ue8m0", [False, True])
def test_config5_forward_backward_at_full_size(ue8m0):
    """128 experts, hidden 4096, intermediate 1408, 131072 routed rows, Zipf(1.0): forward, dgrad-down,
    SwiGLU backward, dgrad-up, both gradient quantizations and both grouped weight gradients."""
    torch.backends.cuda.matmul.allow_tf32 = False
    E, H, I = 128, 4096, 1408
    node, experts, x, probs, rows, counts, (g1, g2) = _build(E, H, I, 131072, 1.0, seed=5, n_empty=0, ue8m0=ue8m0)
    Mpad = sum(rows)
    gen = torch.Generator(device="cuda").manual_seed(55)
    dout = (torch.randn((Mpad, H), generator=gen, device="cuda") * 1e-3).to(torch.bfloat16)
    tag = "config 5" + (" ue8m0" if ue8m0 else "")
    with _Recorder() as rec:
        node.forward(x, probs, rows)
    o1 = _check_forward(rec, node, x, probs, rows, ue8m0, tag)
    x_fp8, x_scale = node.input_fp8, node.input_scale      # cached quantised input, scale a [M, K/128] view

    # launch by launch in the reference's sequence (the SwiGLU backward writing bf16 do1 and o2_s); the node's default, one
    # kernel that writes only their quantized forms, is held against this run at the end
    node.fuse_bwd_swiglu_quant = False
    with _Recorder() as rec:
        dx, pg = node.backward(dout, probs, rows)
    names = [c[0] for c in rec.calls]
    assert names.count("quant_and_transpose_split") == 2 and names.count("m_grouped_fp8_gemm_nt_contiguous") == 2
    assert names.count("fused_swiglu_weighted_bwd") == 1 and names.count("grouped_wgrad") == 2, names
    nz = [e for e, r in enumerate(rows) if r > 0]
    small = min(nz, key=lambda e: rows[e])
    one = [e for e in nz if rows[e] == 128][:1]
    offs = np.concatenate([[0], np.cumsum(rows)]).astype(np.int64)

    def seg(t, e):
        return t[int(offs[e]):int(offs[e + 1])]

    # out_grad: row-wise for dgrad-down, transposed per expert for the down weight gradient, from one read
    qts = rec.named("quant_and_transpose_split")
    g_q, g_s, g_tq, g_ts = qts[0][3]
    assert qts[0][1][0] is dout
    _check_quant_rows(dout, g_q, g_s, rows, ue8m0, f"{tag} quant(dOut)")
    _check_transposed(lambda e: G.from_torch_bf16(seg(dout, e)), g_tq, g_ts, rows, [small] + one, f"{tag} dOut^T")
    gemms = rec.named("m_grouped_fp8_gemm_nt_contiguous")
    _check_grouped_gemm(gemms[0], rows, f"{tag} dgrad-down")
    # SwiGLU backward on the GPU's do2_s: bit-exact do1 and o2_s on the slabs, probs_grad to 1e-5 of its terms
    sb = rec.named("fused_swiglu_weighted_bwd")[0]
    o1_in, do2_s, _ = sb[1][:3]
    do1, pg_rec, o2_s = sb[3]
    assert o1_in is o1 and torch.equal(pg_rec, pg)
    for lo, _, label in _slab_tiles(rows):
        sl = slice(lo, lo + 128)
        edo1, epg, eo2s = O.swiglu_weighted_bwd(G.from_torch_bf16(o1[sl]), G.from_torch_bf16(do2_s[sl]), probs[sl, 0].cpu().numpy())
        msg = G.mismatch_report(G.from_torch_bf16(do1[sl]), edo1, f"{tag} do1, {label}")
        assert not msg, msg
        msg = G.mismatch_report(G.from_torch_bf16(o2_s[sl]), eo2s, f"{tag} o2_s, {label}")
        assert not msg, msg
        terms = (do2_s[sl].float().abs() * (o2_s[sl].float().abs() / probs[sl].clamp_min(1e-30))).sum(dim=1).cpu().numpy()
        assert np.all(np.abs(pg[sl].cpu().numpy() - epg) <= 1e-5 * terms + 1e-30), f"{tag} probs_grad, {label}"
    # do1: row-wise for dgrad-up, transposed per expert for the up+gate weight gradient
    d_q, d_s, d_tq, d_ts = qts[1][3]
    assert qts[1][1][0] is do1
    _check_quant_rows(do1, d_q, d_s, rows, ue8m0, f"{tag} quant(do1)")
    _check_transposed(lambda e: G.from_torch_bf16(seg(do1, e)), d_tq, d_ts, rows, [small] + one, f"{tag} do1^T")
    _check_grouped_gemm(gemms[1], rows, f"{tag} dgrad-up")
    assert gemms[1][1][2] is dx
    # the transposed copies the weight gradients read that were quantized on their own: the cached e4m3 input and o2_s
    tsq = rec.named("fused_transpose_split_quant")
    assert len(tsq) == 2
    by_src = {("fp8" if c[1][0].dtype == torch.float8_e4m3fn else "bf16"): c for c in tsq}
    xt_q, xt_s = by_src["fp8"][3]
    assert by_src["fp8"][1][0] is x_fp8
    _check_transposed(lambda e: (G.from_torch_fp8(seg(x_fp8, e)), seg(_scales_f32(x_scale), e).contiguous().cpu().numpy()), xt_q, xt_s, rows,
                      [small] + one, f"{tag} X^T from e4m3")
    o2t_q, o2t_s = by_src["bf16"][3]
    assert by_src["bf16"][1][0] is o2_s
    _check_transposed(lambda e: G.from_torch_bf16(seg(o2_s, e)), o2t_q, o2t_s, rows, [small] + one, f"{tag} o2_s^T")
    # weight gradients: both grouped launches wrote into zeroed [E, K, N] buffers
    wg = rec.named("grouped_wgrad")
    outs = {tuple(c[1][4].shape): c for c in wg}
    assert set(outs) == {(E, H, 2 * I), (E, I, H)}
    assert outs[(E, H, 2 * I)][1][4].data_ptr() == g1.data_ptr() and outs[(E, I, H)][1][4].data_ptr() == g2.data_ptr()
    _check_grouped_wgrad(outs[(E, H, 2 * I)], rows, f"{tag} dW1")
    _check_grouped_wgrad(outs[(E, I, H)], rows, f"{tag} dW2")
    # the same backward with the SwiGLU backward fused into the quantizations of its results: dx and both weight gradients
    # to the bit, probs_grad (summed per column tile, then over the tiles) to 1e-5 of the magnitudes of its terms
    dw1, dw2 = g1.clone(), g2.clone()
    g1.zero_()
    g2.zero_()
    node.fuse_bwd_swiglu_quant = True
    node.forward(x, probs, rows)
    with _Recorder() as rec:
        dx_f, pg_f = node.backward(dout, probs, rows)
    names = [c[0] for c in rec.calls]
    assert names.count("swiglu_weighted_bwd_quant") == 1 and "fused_swiglu_weighted_bwd" not in names, names
    assert names.count("quant_and_transpose_split") == 1 and names.count("grouped_wgrad") == 2, names
    assert torch.equal(dx_f.view(torch.int16), dx.view(torch.int16)), f"{tag} dx with the fused SwiGLU backward"
    assert torch.equal(g1, dw1) and torch.equal(g2, dw2), f"{tag} weight gradients with the fused SwiGLU backward"
    terms = (do2_s.float().abs() * (o2_s.float().abs() / probs.clamp_min(1e-30))).sum(dim=1)
    assert bool(((pg_f - pg).abs() <= 1e-5 * terms + 1e-30).all()), f"{tag} probs_grad with the fused SwiGLU backward"
