"""Pins the oracle's tensor functions (CPU only) against independent restatements: numpy chains
that follow the reference's un-fused branches, float64 brute force, and invariants of the maths."""
import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G
from tests.test_oracle_codec import _brute_force_encode


def _np_quant_tile(x_f32, pow2=False):
    """One tile, numpy float32 arithmetic + the brute-force encoder: s = amax/448, q = rne(x/s)."""
    amax = np.float32(np.max(np.abs(x_f32))) if x_f32.size else np.float32(0)
    if amax == 0:
        s = np.float32(1)
    else:
        s = np.float32(amax) / np.float32(448.0)
        if pow2:
            s = np.float32(2.0 ** np.ceil(np.log2(np.float64(s))))
    y = (x_f32.astype(np.float32) / s).astype(np.float32)
    return _brute_force_encode(y), s


def _np_quant_1x128(bits, pow2=False):
    x = O.bf16_bits_to_f32(bits)
    M, K = x.shape
    q = np.empty((M, K), np.uint8)
    s = np.empty((M, K // 128), np.float32)
    for r in range(M):
        for b in range(K // 128):
            q[r, b * 128:(b + 1) * 128], s[r, b] = _np_quant_tile(x[r, b * 128:(b + 1) * 128], pow2)
    return q, s


@pytest.mark.parametrize("pow2", [False, True])
def test_quant_1x128_brute_force(pow2):
    bits = G.bf16_normal((24, 384), seed=1, outlier_frac=5e-3, outlier_scale=100.0)
    bits[3, :128] = 0            # an all-zero tile
    bits[4, 128:256] = 0x8000    # all negative zero
    q, s = O.quant_1x128(bits, 0, pow2)
    eq, es = _np_quant_1x128(bits, pow2)
    assert np.array_equal(q, eq) and np.array_equal(s, es)
    assert s[3, 0] == 1.0 and (q[3, :128] == 0).all() and (q[4, 128:256] == 0x80).all()
    # the transposed scale layout holds the same numbers
    q2, s2 = O.quant_1x128(bits, 1, pow2)
    assert np.array_equal(q2, q) and np.array_equal(s2, s.T)


def test_quant_1x128_invariants():
    bits = G.bf16_normal((64, 512), seed=2, outlier_frac=1e-3, outlier_scale=100.0)
    q, s = O.quant_1x128(bits, 0)
    # the amax element of every tile maps to +-448 and s*448 reproduces amax to an ulp
    x = O.bf16_bits_to_f32(bits).reshape(64, 4, 128)
    amax = np.abs(x).max(axis=-1)
    assert ((q.reshape(64, 4, 128) & 0x7F).max(axis=-1) == 0x7E).all()
    assert np.all(np.abs(s * np.float32(448) - amax) <= np.spacing(amax))
    # scaling the input by a power of two leaves the bytes alone and scales s
    x4 = O.f32_to_bf16_bits(O.bf16_bits_to_f32(bits) * np.float32(4))
    q4, s4 = O.quant_1x128(x4, 0)
    assert np.array_equal(q4, q) and np.array_equal(s4, s * 4)
    # tiles are independent: permuting rows permutes outputs
    perm = np.random.default_rng(0).permutation(64)
    qp, sp = O.quant_1x128(bits[perm], 0)
    assert np.array_equal(qp, q[perm]) and np.array_equal(sp, s[perm])
    # dequantised values are within half an e4m3 step of the input (relative 2^-4 for normals)
    deq = O.bf16_bits_to_f32(O.act_dequant(q, s, 0))
    xf = O.bf16_bits_to_f32(bits)
    big = np.abs(xf) > np.repeat(s, 128, axis=1) * 2.0**-6
    assert np.max(np.abs(deq - xf)[big] / np.abs(xf)[big]) <= 2.0**-4 + 2.0**-8


@pytest.mark.parametrize("pow2", [False, True])
def test_quant_128x128_brute_force_and_transpose_identity(pow2):
    bits = G.bf16_normal((256, 384), seed=3, std=0.02, outlier_frac=1e-3, outlier_scale=50.0)
    q, s, qt, st = O.quant_128x128(bits, want=(True, True), pow2=pow2)
    x = O.bf16_bits_to_f32(bits)
    for rb in range(2):
        for cb in range(3):
            eq, es = _np_quant_tile(x[rb * 128:(rb + 1) * 128, cb * 128:(cb + 1) * 128], pow2)
            assert np.array_equal(q[rb * 128:(rb + 1) * 128, cb * 128:(cb + 1) * 128], eq)
            assert s[rb, cb] == es
    # quant128(W^T) == quant128(W)^T, bytes and scales (transformers/fp8_utils.py:110,123)
    q2, s2, _, _ = O.quant_128x128(np.ascontiguousarray(bits.T), pow2=pow2)
    assert np.array_equal(q2, q.T) and np.array_equal(s2, s.T)
    assert np.array_equal(qt, q.T) and np.array_equal(st, s.T)


def test_quant_transpose_is_two_quantizations():
    bits = G.bf16_normal((256, 384), seed=4, outlier_frac=1e-3, outlier_scale=100.0)
    for lay in (0, 1):
        q, s, qt, st = O.quant_transpose(bits, scale_layout=lay)
        eq, es = _np_quant_1x128(bits)
        eqt, est = _np_quant_1x128(np.ascontiguousarray(bits.T))
        assert np.array_equal(q, eq) and np.array_equal(qt, eqt)
        assert np.array_equal(s, es.T if lay else es) and np.array_equal(st, est.T if lay else est)
        _, _, qt2, st2 = O.quant_transpose(bits, scale_layout=lay, want_row=False)
        assert np.array_equal(qt2, qt) and np.array_equal(st2, st)


@pytest.mark.parametrize("transpose", [False, True])
def test_stack_transpose_quant_is_the_unfused_chain(transpose):
    """ernie token_dispatcher/fp8_utils.py:276-287: stack -> transpose([0,2,1]) -> reshape -> quant128."""
    ws = [G.bf16_normal((128, 256), seed=10 + e, std=0.02) for e in range(3)]
    q, s = O.stack_transpose_quant(ws, transpose=transpose)
    stacked = np.stack(ws)
    if transpose:
        stacked = np.ascontiguousarray(stacked.transpose(0, 2, 1))
    flat = stacked.reshape(-1, stacked.shape[-1])
    eq, es, _, _ = O.quant_128x128(flat)
    assert np.array_equal(q, eq) and np.array_equal(s, es)


def test_swiglu_weighted_quant_chain():
    M, I = 16, 256
    bits = G.bf16_normal((M, 2 * I), seed=5, std=2.0)
    probs = np.random.default_rng(5).random(M, dtype=np.float32)
    q, s, o2 = O.swiglu_weighted_quant(bits, probs, 0, False, return_o2=True)
    # float64 restatement of the un-fused chain; bf16 results may differ by one ulp at most
    x = O.bf16_bits_to_f32(bits).astype(np.float64)
    g, u = x[:, :I], x[:, I:]
    sw = O.bf16_bits_to_f32(O.f32_to_bf16_bits((g / (1 + np.exp(-g)) * u).astype(np.float32)))
    ref = O.f32_to_bf16_bits((sw.astype(np.float64) * probs[:, None]).astype(np.float32))
    d = np.abs(o2.astype(np.int32) - ref.astype(np.int32))
    assert d.max() <= 1 and (d == 0).mean() > 0.98
    # gate is the FIRST half: swapping halves changes the result
    swapped = np.concatenate([bits[:, I:], bits[:, :I]], axis=1)
    assert not np.array_equal(O.swiglu_weighted_quant(swapped, probs, 0, False, return_o2=True)[2], o2)
    # the quantised output is exactly the 1x128 quantization of those activations
    eq, es = O.quant_1x128(o2, 0)
    assert np.array_equal(q, eq) and np.array_equal(s, es)
    # probs == 1 is the same as no probs (dense-MLP chain)
    qa, sa = O.swiglu_weighted_quant(bits, np.ones(M, np.float32))
    qb, sb = O.swiglu_weighted_quant(bits, None)
    assert np.array_equal(qa, qb) and np.array_equal(sa, sb)


def test_transpose_split_quant_is_the_unfused_chain():
    """ernie token_dispatcher/fp8_utils.py:1199-1210: per expert x_e.T.contiguous() -> quant 1x128 (scale^T)."""
    rows = [256, 0, 128]
    K = 256
    bits = G.bf16_normal((sum(rows), K), seed=6, outlier_frac=1e-3, outlier_scale=100.0)
    qs, ss = O.transpose_split_quant(bits, None, rows, pow2=True)
    off = 0
    for e, r in enumerate(rows):
        assert qs[e].shape == (K, r) and ss[e].shape == (r // 128, K)
        if r:
            eq, es = O.quant_1x128(np.ascontiguousarray(bits[off:off + r].T), 1, True)
            assert np.array_equal(qs[e], eq) and np.array_equal(ss[e], es)
        off += r
    # fp8 input: dequantise to bf16 first, either scale layout
    xq, xs = O.quant_1x128(bits, 0)
    deq = O.act_dequant(xq, xs, 0)
    q1, s1 = O.transpose_split_quant(xq, xs, rows, pow2=True)
    q2, s2 = O.transpose_split_quant(deq, None, rows, pow2=True)
    q3, s3 = O.transpose_split_quant(xq, np.ascontiguousarray(xs.T), rows, pow2=True, xs_layout=1)
    for e in range(3):
        assert np.array_equal(q1[e], q2[e]) and np.array_equal(s1[e], s2[e])
        assert np.array_equal(q1[e], q3[e]) and np.array_equal(s1[e], s3[e])


def test_dequant_block_broadcast_kats():
    """Shape of the reference's KATs (test_coverage_hf_checkpoint_dequant.py:272-288) at the
    128-wide block this path uses: a scale grid is broadcast over blocks, trailing partial blocks
    are cropped."""
    one = 0x38
    q = np.full((256, 384), one, np.uint8)
    s = np.array([[1.0, 2.0, 4.0], [0.5, 8.0, 16.0]], np.float32)
    out = O.bf16_bits_to_f32(O.weight_dequant(q, s))
    assert np.array_equal(out, np.repeat(np.repeat(s, 128, 0), 128, 1))
    q = np.full((130, 257), one, np.uint8)
    s = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    out = O.bf16_bits_to_f32(O.weight_dequant(q, s))
    assert out.shape == (130, 257) and out[127, 255] == 2 and out[128, 256] == 6 and out[129, 0] == 4
    # 1x128: both scale layouts
    qa = np.full((4, 256), one, np.uint8)
    sa = np.arange(8, dtype=np.float32).reshape(4, 2) + 1
    assert np.array_equal(O.bf16_bits_to_f32(O.act_dequant(qa, sa, 0)), np.repeat(sa, 128, 1))
    assert np.array_equal(O.act_dequant(qa, np.ascontiguousarray(sa.T), 1), O.act_dequant(qa, sa, 0))


def test_swiglu_bwd_against_finite_differences():
    M, I = 6, 8
    rng = np.random.default_rng(7)
    o1 = O.f32_to_bf16_bits(rng.standard_normal((M, 2 * I)).astype(np.float32))
    do2_s = O.f32_to_bf16_bits(rng.standard_normal((M, I)).astype(np.float32))
    probs = rng.random(M, dtype=np.float32) + 0.1
    do1, pg, o2s = O.swiglu_weighted_bwd(o1, do2_s, probs)
    x = O.bf16_bits_to_f32(o1).astype(np.float64)
    d = O.bf16_bits_to_f32(do2_s).astype(np.float64)

    def loss(xv, pv):
        g, u = xv[:, :I], xv[:, I:]
        return np.sum(d * (g / (1 + np.exp(-g)) * u) * pv[:, None])

    num = np.zeros_like(x)
    eps = 1e-6
    for i in range(M):
        for j in range(2 * I):
            xp, xm = x.copy(), x.copy()
            xp[i, j] += eps
            xm[i, j] -= eps
            num[i, j] = (loss(xp, probs.astype(np.float64)) - loss(xm, probs.astype(np.float64))) / (2 * eps)
    got = O.bf16_bits_to_f32(do1).astype(np.float64)
    # bf16 roundings of do2 and of the result: 2^-7 relative plus a small absolute floor
    assert np.all(np.abs(got - num) <= 2.0**-6 * np.abs(num) + 1e-3)
    # probs_grad = d loss / d probs = sum_j do2_s * swiglu (with swiglu rounded to bf16)
    g, u = x[:, :I], x[:, I:]
    sw = g / (1 + np.exp(-g)) * u
    assert np.all(np.abs(pg - (d * sw).sum(1)) <= 2.0**-7 * np.abs(d * sw).sum(1) + 1e-6)
    # o2_s is the forward activation times probs (checked at a quantisable width)
    o1w = O.f32_to_bf16_bits(rng.standard_normal((M, 256)).astype(np.float32))
    dw = O.f32_to_bf16_bits(rng.standard_normal((M, 128)).astype(np.float32))
    _, _, o2sw = O.swiglu_weighted_bwd(o1w, dw, probs)
    _, _, o2 = O.swiglu_weighted_quant(o1w, probs, return_o2=True)
    assert np.array_equal(o2sw, o2)


def _rand_codes(shape, seed, lo=-3, hi=3):
    v = np.random.default_rng(seed).integers(lo, hi + 1, shape).astype(np.float32)
    return O.e4m3_encode_array(v), v


def test_gemm_exact_integer_case_and_scale_indexing():
    M, N, K = 16, 256, 384
    a, av = _rand_codes((M, K), 1)
    b, bv = _rand_codes((N, K), 2)
    sa = np.ones((M, 3), np.float32)
    sb = np.ones((2, 3), np.float32)
    out = O.bf16_bits_to_f32(O.gemm_nt(a, sa, b, sb))
    assert np.array_equal(out, O.bf16_bits_to_f32(O.f32_to_bf16_bits((av @ bv.T).astype(np.float32))))
    # distinct power-of-two scales per (row, k-block) and per (n-block, k-block): still exact
    sa = (2.0 ** np.random.default_rng(3).integers(-3, 4, (M, 3))).astype(np.float32)
    sb = (2.0 ** np.random.default_rng(4).integers(-3, 4, (2, 3))).astype(np.float32)
    exact = (av * np.repeat(sa, 128, 1)) @ (bv * np.repeat(np.repeat(sb, 128, 0), 128, 1)).T
    for lay, s_in in ((0, sa), (1, np.ascontiguousarray(sa.T))):
        out = O.bf16_bits_to_f32(O.gemm_nt(a, s_in, b, sb, sa_layout=lay))
        assert np.array_equal(out, O.bf16_bits_to_f32(O.f32_to_bf16_bits(exact.astype(np.float32))))
        ref = O.bf16_bits_to_f32(O.gemm_nt(a, s_in, b, sb, sa_layout=lay, dequant_ref=True))
        assert np.array_equal(out, ref)


def test_gemm_block_accumulation_vs_float64_dequant_matmul():
    M, N, K = 32, 128, 512
    xa = G.bf16_normal((M, K), seed=5)
    wb = G.bf16_normal((N, K), seed=6, std=0.02, outlier_frac=1e-3, outlier_scale=50.0)
    a, sa = O.quant_1x128(xa, 0)
    b, sb, _, _ = O.quant_128x128(wb)
    blk = O.bf16_bits_to_f32(O.gemm_nt(a, sa, b, sb))
    ref = O.bf16_bits_to_f32(O.gemm_nt(a, sa, b, sb, dequant_ref=True))
    np_ref = (O.e4m3_decode_np(a).astype(np.float64) * np.repeat(sa, 128, 1)) @ \
             (O.e4m3_decode_np(b).astype(np.float64) * np.repeat(np.repeat(sb, 128, 0), 128, 1)).T
    assert np.array_equal(ref, O.bf16_bits_to_f32(O.f32_to_bf16_bits(np_ref.astype(np.float32))))
    assert G.rel_fro(blk, ref) < 1e-4
    # and the quantised product tracks the bf16 product to FP8 accuracy
    full = O.bf16_bits_to_f32(xa).astype(np.float64) @ O.bf16_bits_to_f32(wb).astype(np.float64).T
    assert G.rel_fro(blk, full) < 0.06


def test_grouped_gemms_equal_per_expert_dense():
    E, N, K = 3, 128, 256
    rows = [128, 0, 256]
    Mtot = sum(rows)
    a, sa = O.quant_1x128(G.bf16_normal((Mtot, K), seed=7), 0)
    b = np.empty((E, N, K), np.uint8)
    sb = np.empty((E, 1, 2), np.float32)
    for e in range(E):
        b[e], sb[e], _, _ = O.quant_128x128(G.bf16_normal((N, K), seed=8 + e, std=0.02))
    m_idx = np.repeat(np.arange(E, dtype=np.int32), rows)
    out = O.grouped_gemm_nt_contiguous(a, sa, b, sb, m_idx)
    off = 0
    for e, r in enumerate(rows):
        if r:
            assert np.array_equal(out[off:off + r], O.gemm_nt(a[off:off + r], sa[off:off + r], b[e], sb[e]))
        off += r
    # masked layout == contiguous on the valid rows; the rest untouched
    Mmax = 256
    am = np.zeros((E, Mmax, K), np.uint8)
    sam = np.ones((E, Mmax, 2), np.float32)
    off = 0
    for e, r in enumerate(rows):
        am[e, :r], sam[e, :r] = a[off:off + r], sa[off:off + r]
        off += r
    init = np.full((E, Mmax, N), 0x4000, np.uint16)
    outm = O.grouped_gemm_nt_masked(am, sam, b, sb, np.array(rows, np.int32), out=init.copy())
    off = 0
    for e, r in enumerate(rows):
        assert np.array_equal(outm[e, :r], out[off:off + r]) and np.array_equal(outm[e, r:], init[e, r:])
        off += r


def test_wgrad_is_dequant_matmul_with_accumulate():
    Kin, N, M = 64, 48, 256
    x = G.bf16_normal((M, Kin), seed=9)
    d = G.bf16_normal((M, N), seed=10, std=1e-3)
    a_t, sa_t = O.quant_1x128(np.ascontiguousarray(x.T), 1)
    b_t, sb_t = O.quant_1x128(np.ascontiguousarray(d.T), 1)
    out = O.gemm_nt_1d1d_f32(a_t, sa_t, b_t, sb_t)
    ad = O.e4m3_decode_np(a_t).astype(np.float64) * np.repeat(sa_t.T, 128, 1)
    bd = O.e4m3_decode_np(b_t).astype(np.float64) * np.repeat(sb_t.T, 128, 1)
    assert G.rel_fro(out, ad @ bd.T) < 1e-6
    base = np.random.default_rng(0).standard_normal((Kin, N)).astype(np.float32)
    acc = O.gemm_nt_1d1d_f32(a_t, sa_t, b_t, sb_t, out=base)
    assert np.allclose(acc, base + out, rtol=0, atol=1e-6 * np.abs(out).max() + 1e-7)
    # it approximates dW = x^T . dout
    full = O.bf16_bits_to_f32(x).astype(np.float64).T @ O.bf16_bits_to_f32(d).astype(np.float64)
    assert G.rel_fro(out, full) < 0.06


def test_moe_permute_unpermute_invariants():
    """The numpy restatement of moe_permute / moe_unpermute (parity unpinned): segments start at the
    padded prefix sums, rows of an expert keep token order, padding rows are zero, the way back sums
    the copies (exact for small integers) and returns the probabilities to their slots."""
    rng = np.random.default_rng(0)
    T, H, topk, E = 50, 16, 3, 5
    rm = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    rm[rng.random(rm.shape) < 0.2] = -1
    counts = [int((rm == e).sum()) for e in range(E)]
    probs = rng.random(rm.shape).astype(np.float32)
    xv = rng.integers(-4, 5, size=(T, H)).astype(np.float32)
    x = O.f32_to_bf16_bits(xv)
    ox, rowmap, op, _ = O.moe_permute(x, None, rm, probs, E, counts, 8)
    padded = [(c + 7) // 8 * 8 for c in counts]
    starts = np.concatenate([[0], np.cumsum(padded)])
    assert ox.shape[0] == starts[-1]
    for e in range(E):
        col = rowmap[:, e][rowmap[:, e] >= 0]
        assert len(col) == counts[e] and (col == starts[e] + np.arange(counts[e])).all()
        assert not ox[starts[e] + counts[e]:starts[e + 1]].any() and not op[starts[e] + counts[e]:starts[e + 1]].any()
    for t in range(T):
        for k in range(topk):
            if rm[t, k] >= 0:
                assert (ox[rowmap[t, rm[t, k]]] == x[t]).all() and op[rowmap[t, rm[t, k]], 0] == probs[t, k]
    back, pb = O.moe_unpermute(ox, rowmap, rm, op, T, E)
    assert (O.bf16_bits_to_f32(back) == xv * (rm >= 0).sum(axis=1, keepdims=True)).all()
    assert (pb == np.where(rm >= 0, probs, 0)).all()


def test_moe_permute_row_order_is_the_in_repo_permute_fast():
    """cli/train/deepseek_v3_pretrain/moe_utils.py:57-88 states the un-fused permutation in plain tensor
    operations: for expert 0, 1, ... the flat (token-major) positions of the routing map that name the
    expert, in ascending order; token = position // topk; rows and probabilities are gathered in that order.
    Without padding (alignment 1) the restated operator must give exactly that."""
    rng = np.random.default_rng(1)
    T, H, topk, E = 64, 8, 4, 6
    rm = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    counts = [int((rm == e).sum()) for e in range(E)]
    probs = rng.random(rm.shape).astype(np.float32)
    x = O.f32_to_bf16_bits(rng.standard_normal((T, H)).astype(np.float32))
    flat = rm.reshape(-1)
    prob_idx = np.concatenate([np.nonzero(flat == e)[0] for e in range(E)])       # topk_to_permuted_indices
    token_idx = prob_idx // topk
    ox, rowmap, op, _ = O.moe_permute(x, None, rm, probs, E, counts, 1)
    assert np.array_equal(ox, x[token_idx])                                     # permute_fast: index_select
    assert np.array_equal(op[:, 0], probs.reshape(-1)[prob_idx])                # the probs gathered the same way
    # the row map is the inverse of that order
    for r, (t, p) in enumerate(zip(token_idx, prob_idx)):
        assert rowmap[t, flat[p]] == r
    # unpermute_fast (:90-130) scatter-adds the permuted rows back to their tokens: small integers make it exact
    xi = rng.integers(-3, 4, size=(T, H)).astype(np.float32)
    oxi, rowmap, opi, _ = O.moe_permute(O.f32_to_bf16_bits(xi), None, rm, probs, E, counts, 1)
    back, _ = O.moe_unpermute(oxi, rowmap, rm, opi, T, E)
    ref = np.zeros((T, H), np.float32)
    np.add.at(ref, token_idx, O.bf16_bits_to_f32(oxi))
    assert np.array_equal(O.bf16_bits_to_f32(back), ref)
