"""Writes tests/golden/pf8_golden.npz: small seeded inputs and the outputs the CPU oracle gives for them,
one group per operator of the path.  The oracle is pinned by the reference's known-answer vectors, closed
forms and invariants (tests/test_oracle_*.py); these fixtures freeze its outputs, so that a later change of
the oracle or of a kernel that alters a single bit shows up against committed data.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import pf8_oracle as O  # noqa: E402
from tests import _gen as G  # noqa: E402


def build():
    f = {}
    # activations with outliers and one all-zero tile
    x = G.bf16_normal((128, 256), seed=101, outlier_frac=2e-3, outlier_scale=80.0)
    x[5, 128:256] = 0
    f["act_x"] = x
    for pow2 in (0, 1):
        q, s = O.quant_1x128(x, 0, pow2=bool(pow2))
        f[f"quant_1x128_p{pow2}_q"], f[f"quant_1x128_p{pow2}_s"] = q, s
    q, s = O.quant_1x128(x, 1)
    f["quant_1x128_layout1_s"] = s
    qr, sr, qt, st = O.quant_transpose(x, 1)
    f["quant_transpose_q"], f["quant_transpose_s"], f["quant_transpose_qt"], f["quant_transpose_st"] = qr, sr, qt, st
    # weights
    w = G.bf16_normal((256, 256), seed=102, std=0.03)
    f["weight_w"] = w
    q, s, qt, st = O.quant_128x128(w, want=(True, True))
    f["quant_128x128_q"], f["quant_128x128_s"], f["quant_128x128_qt"], f["quant_128x128_st"] = q, s, qt, st
    w2 = G.bf16_normal((256, 256), seed=103, std=0.05)
    f["weight_w2"] = w2
    for tr in (0, 1):
        q, s = O.stack_transpose_quant([w, w2], transpose=bool(tr))
        f[f"stack_quant_t{tr}_q"], f[f"stack_quant_t{tr}_s"] = q, s
    # SwiGLU + requant and its backward
    o1 = G.bf16_normal((128, 512), seed=104, std=1.5)
    probs = (np.random.default_rng(105).random(128, dtype=np.float32) * 0.5 + 0.25).astype(np.float32)
    f["swiglu_o1"], f["swiglu_probs"] = o1, probs
    for pow2 in (0, 1):
        q, s, o2 = O.swiglu_weighted_quant(o1, probs, 0, bool(pow2), return_o2=True)
        f[f"swiglu_quant_p{pow2}_q"], f[f"swiglu_quant_p{pow2}_s"] = q, s
    f["swiglu_quant_o2"] = o2
    do2 = G.bf16_normal((128, 256), seed=106, std=0.01)
    f["swiglu_bwd_do2"] = do2
    do1, pg, o2s = O.swiglu_weighted_bwd(o1, do2, probs)
    f["swiglu_bwd_do1"], f["swiglu_bwd_pg"], f["swiglu_bwd_o2s"] = do1, pg, o2s
    # transpose + split + quant: bf16 source and e4m3 source
    rows = np.array([128, 0, 256], np.int64)
    xs3 = G.bf16_normal((384, 256), seed=107, outlier_frac=2e-3, outlier_scale=50.0)
    f["split_x"], f["split_rows"] = xs3, rows
    qs, ss = O.transpose_split_quant(xs3, None, [int(r) for r in rows], True)
    for e in (0, 2):
        f[f"split_bf16_q{e}"], f[f"split_bf16_s{e}"] = qs[e], ss[e]
    xq, xsc = O.quant_1x128(xs3, 0)
    qs, ss = O.transpose_split_quant(xq, xsc, [int(r) for r in rows], True)
    for e in (0, 2):
        f[f"split_fp8_q{e}"], f[f"split_fp8_s{e}"] = qs[e], ss[e]
    # dequantizers (ragged weight)
    f["act_dequant_out"] = O.act_dequant(f["quant_1x128_p0_q"], f["quant_1x128_p0_s"], 0)
    rng = np.random.default_rng(108)
    dq = rng.integers(0, 256, (200, 300)).astype(np.uint8)
    dsc = ((rng.random((2, 3), dtype=np.float32) + 0.5) * np.float32(0.01)).astype(np.float32)
    f["weight_dequant_q"], f["weight_dequant_s"] = dq, dsc
    f["weight_dequant_out"] = O.weight_dequant(dq, dsc)
    e8 = rng.integers(118, 136, (2, 3)).astype(np.uint8)
    f["block_dequant_e8"] = e8
    f["block_dequant_out"] = O.block_dequant(dq, e8, "ue8m0", (0, 1), (128, 128), out="bf16")
    f["scales_pow2"] = np.exp2(rng.integers(-20, 20, 64)).astype(np.float32)
    f["scales_ue8m0"] = O.scales_to_ue8m0(f["scales_pow2"])
    # GEMMs
    a, sa = O.quant_1x128(G.bf16_normal((256, 256), seed=109), 0)
    b, sb, _, _ = O.quant_128x128(G.bf16_normal((256, 256), seed=110, std=0.05))
    f["gemm_a"], f["gemm_sa"], f["gemm_b"], f["gemm_sb"] = a, sa, b, sb
    f["gemm_nt_out"] = O.gemm_nt(a, sa, b, sb)
    b2, sb2, _, _ = O.quant_128x128(G.bf16_normal((256, 256), seed=111, std=0.05))
    f["gemm_b2"], f["gemm_sb2"] = b2, sb2
    m_idx = np.array([0] * 128 + [1] * 128, np.int32)
    f["grouped_contig_out"] = O.grouped_gemm_nt_contiguous(a, sa, np.stack([b, b2]), np.stack([sb, sb2]), m_idx)
    masked = np.array([100, 37], np.int32)
    f["grouped_masked_m"] = masked
    f["grouped_masked_out"] = O.grouped_gemm_nt_masked(a.reshape(2, 128, 256), sa.reshape(2, 128, 2), np.stack([b, b2]), np.stack([sb, sb2]), masked)
    at, sat = O.quant_1x128(G.bf16_normal((128, 256), seed=112), 1)     # [Ka, M] with scales [M/128, Ka]
    bt, sbt = O.quant_1x128(G.bf16_normal((256, 256), seed=113, std=0.01), 1)
    f["wgrad_at"], f["wgrad_sat"], f["wgrad_bt"], f["wgrad_sbt"] = at, sat, bt, sbt
    f["wgrad_out"] = O.gemm_nt_1d1d_f32(at, sat, bt, sbt)
    return f


if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "pf8_golden.npz")
    np.savez_compressed(out, **build())
    print("wrote", out, os.path.getsize(out), "bytes")
