"""ctypes front end of the CPU oracle (libpf8_oracle.so) on numpy arrays.

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the CPU-baseline leg of the
benchmark.  The product package never imports it.

bf16 tensors are numpy uint16 bit patterns, e4m3 tensors are numpy uint8 codes, scales float32.
Each wrapper names the C function it calls; the reference citations live in pf8_oracle.c.

A few restatements at the end of this file are plain numpy, not C:
  block_dequant              pinned by the reference's own known-answer vectors
                             (tests/test_oracle_dequant.py)
  scales_to_ue8m0            pinned as the inverse of the UE8M0 decode table above, itself pinned by
                             those vectors (tests/test_oracle_dequant.py)
  moe_permute / moe_unpermute  PARITY UNPINNED: no test, fixture or importable implementation of
                             the operators exists in the reference; checked only against the
                             invariants their call sites rely on (tests/test_oracle_ops.py)
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libpf8_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (make -C oracle)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []), stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.pf8o_e4m3_decode.restype = C.c_float
        _lib.pf8o_e4m3_decode.argtypes = [C.c_uint8]
        _lib.pf8o_e4m3_encode.restype = C.c_uint8
        _lib.pf8o_e4m3_encode.argtypes = [C.c_float]
        _lib.pf8o_bf16_to_f32.restype = C.c_float
        _lib.pf8o_bf16_to_f32.argtypes = [C.c_uint16]
        _lib.pf8o_f32_to_bf16.restype = C.c_uint16
        _lib.pf8o_f32_to_bf16.argtypes = [C.c_float]
        _lib.pf8o_expf.restype = C.c_float
        _lib.pf8o_expf.argtypes = [C.c_float]
        _lib.pf8o_silu.restype = C.c_float
        _lib.pf8o_silu.argtypes = [C.c_float]
        _lib.pf8o_scale_from_amax.restype = C.c_float
        _lib.pf8o_scale_from_amax.argtypes = [C.c_float, C.c_int]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    a = np.ascontiguousarray(a)
    assert a.dtype == dt, (a.dtype, dt)
    return a


I64 = C.c_int64

# ---------------------------------------------------------------------------------------------
# numpy-side helpers (independent of the C code; used to cross-check it)
# ---------------------------------------------------------------------------------------------


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns, round-to-nearest-even (numpy restatement)."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (b & 0x7FFFFFFF) > 0x7F800000
    r = (b + 0x7FFF + ((b >> 16) & 1)) >> 16
    r = np.where(nan, (b >> 16) | 0x40, r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def e4m3_table() -> np.ndarray:
    """The 256-entry decode table from the closed form (float64)."""
    t = np.empty(256, dtype=np.float64)
    for c in range(256):
        e, m = (c >> 3) & 0xF, c & 7
        if e == 0xF and m == 7:
            v = np.nan
        elif e == 0:
            v = m * 2.0**-9
        else:
            v = (1 + m / 8.0) * 2.0 ** (e - 7)
        t[c] = -v if c & 0x80 else v
    return t


def e4m3_decode_np(q: np.ndarray) -> np.ndarray:
    return e4m3_table().astype(np.float32)[np.ascontiguousarray(q, dtype=np.uint8)]


# ---------------------------------------------------------------------------------------------
# scalar entry points
# ---------------------------------------------------------------------------------------------


def e4m3_decode(c: int) -> float:
    return lib().pf8o_e4m3_decode(c)


def e4m3_encode(v: float) -> int:
    return lib().pf8o_e4m3_encode(float(v))


def expf(x: float) -> float:
    return lib().pf8o_expf(float(x))


def silu(x: float) -> float:
    return lib().pf8o_silu(float(x))


def scale_from_amax(amax: float, pow2: bool = False) -> float:
    return lib().pf8o_scale_from_amax(float(amax), int(pow2))


def _array_fn(name, v, out_dtype):
    flat = np.ascontiguousarray(v, dtype=np.float32).ravel()
    out = np.empty(flat.size, out_dtype)
    getattr(lib(), name)(_p(flat), I64(flat.size), _p(out))
    return out.reshape(np.shape(v))


def e4m3_encode_array(v):
    return _array_fn("pf8o_e4m3_encode_array", v, np.uint8)


def expf_array(v):
    return _array_fn("pf8o_expf_array", v, np.float32)


def silu_array(v):
    return _array_fn("pf8o_silu_array", v, np.float32)


def f32_to_bf16_array(v):
    return _array_fn("pf8o_f32_to_bf16_array", v, np.uint16)


def check_reciprocal_division(pow2=False, min_scale=1.0e-30):
    """Exhaustive sweep of the reciprocal-and-residual division over every (bf16 amax, bf16 x <= amax) pair:
    returns (pairs, pairs whose e4m3 code differs from the IEEE divide's, pairs whose fp32 quotient differs)."""
    out = np.zeros(3, np.int64)
    lib().pf8o_check_reciprocal_division(int(pow2), C.c_float(min_scale), _p(out))
    return int(out[0]), int(out[1]), int(out[2])


def div_encode_array(x, s):
    """e4m3_encode(x / s) element-wise with IEEE fp32 division."""
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    s = np.ascontiguousarray(s, dtype=np.float32).ravel()
    out = np.empty(x.size, np.uint8)
    lib().pf8o_div_encode_array(_p(x), _p(s), I64(x.size), _p(out))
    return out


# ---------------------------------------------------------------------------------------------
# tensor entry points
# ---------------------------------------------------------------------------------------------


def quant_1x128(x, scale_layout=0, pow2=False):
    """pf8o_quant_1x128: x uint16[M,K] -> (q uint8[M,K], s float32 [M,K/128] or [K/128,M])."""
    x = _c(x, np.uint16)
    M, K = x.shape
    assert K % 128 == 0
    q = np.empty((M, K), np.uint8)
    s = np.empty((M, K // 128) if scale_layout == 0 else (K // 128, M), np.float32)
    lib().pf8o_quant_1x128(_p(x), I64(M), I64(K), I64(K), _p(q), _p(s), int(scale_layout), int(pow2))
    return q, s


def quant_128x128(w, want=(True, False), pow2=False):
    """pf8o_quant_128x128: returns (q, s, qt, st); entries not wanted are None."""
    w = _c(w, np.uint16)
    R, Cc = w.shape
    assert R % 128 == 0 and Cc % 128 == 0
    q = s = qt = st = None
    if want[0]:
        q, s = np.empty((R, Cc), np.uint8), np.empty((R // 128, Cc // 128), np.float32)
    if want[1]:
        qt, st = np.empty((Cc, R), np.uint8), np.empty((Cc // 128, R // 128), np.float32)
    lib().pf8o_quant_128x128(_p(w), I64(R), I64(Cc), _p(q), _p(s), _p(qt), _p(st), int(pow2))
    return q, s, qt, st


def quant_transpose(x, scale_layout=1, pow2=False, want_row=True):
    """pf8o_quant_transpose: (q[M,K], s, qt[K,M], st)."""
    x = _c(x, np.uint16)
    M, K = x.shape
    assert M % 128 == 0 and K % 128 == 0
    q = s = None
    if want_row:
        q = np.empty((M, K), np.uint8)
        s = np.empty((K // 128, M) if scale_layout else (M, K // 128), np.float32)
    qt = np.empty((K, M), np.uint8)
    st = np.empty((M // 128, K) if scale_layout else (K, M // 128), np.float32)
    lib().pf8o_quant_transpose(_p(x), I64(M), I64(K), _p(q), _p(s), _p(qt), _p(st), int(scale_layout), int(pow2))
    return q, s, qt, st


def stack_transpose_quant(w_list, transpose=False, pow2=False):
    ws = [_c(w, np.uint16) for w in w_list]
    E = len(ws)
    R, Cc = ws[0].shape
    ptrs = (C.c_void_p * E)(*[w.ctypes.data for w in ws])
    if transpose:
        q, s = np.empty((E * Cc, R), np.uint8), np.empty((E * Cc // 128, R // 128), np.float32)
    else:
        q, s = np.empty((E * R, Cc), np.uint8), np.empty((E * R // 128, Cc // 128), np.float32)
    lib().pf8o_stack_transpose_quant(ptrs, int(E), I64(R), I64(Cc), int(transpose), _p(q), _p(s), int(pow2))
    return q, s


def swiglu_weighted_quant(o1, probs=None, scale_layout=0, pow2=False, return_o2=False):
    o1 = _c(o1, np.uint16)
    M, I2 = o1.shape
    I = I2 // 2
    assert I % 128 == 0
    if probs is not None:
        probs = _c(probs, np.float32)
        assert probs.shape == (M,)
    q = np.empty((M, I), np.uint8)
    s = np.empty((M, I // 128) if scale_layout == 0 else (I // 128, M), np.float32)
    o2 = np.empty((M, I), np.uint16)
    lib().pf8o_swiglu_weighted_quant(_p(o1), _p(probs), I64(M), I64(I), _p(q), _p(s), int(scale_layout), int(pow2), _p(o2))
    return (q, s, o2) if return_o2 else (q, s)


def act_dequant(q, s, scale_layout=0):
    q = _c(q, np.uint8)
    s = _c(s, np.float32)
    M, K = q.shape
    out = np.empty((M, K), np.uint16)
    lib().pf8o_act_dequant(_p(q), _p(s), int(scale_layout), I64(M), I64(K), _p(out))
    return out


def weight_dequant(q, s):
    q = _c(q, np.uint8)
    s = _c(s, np.float32)
    R, Cc = q.shape
    assert s.shape == ((R + 127) // 128, (Cc + 127) // 128)
    out = np.empty((R, Cc), np.uint16)
    lib().pf8o_weight_dequant(_p(q), _p(s), I64(R), I64(Cc), _p(out))
    return out


def transpose_split_quant(x, xs, rows, pow2=False, xs_layout=0):
    """pf8o_transpose_split_quant -> (list of qt[e] [K,M_e], list of st[e] [M_e/128,K])."""
    is_fp8 = x.dtype == np.uint8
    x = np.ascontiguousarray(x)
    Mtot, K = x.shape
    rows = np.asarray(rows, dtype=np.int64)
    assert rows.sum() == Mtot and (rows % 128 == 0).all()
    if is_fp8:
        xs = _c(xs, np.float32)
        assert xs.shape == ((Mtot, K // 128) if xs_layout == 0 else (K // 128, Mtot))
    qt = np.empty(K * Mtot, np.uint8)
    st = np.empty((Mtot // 128) * K, np.float32)
    lib().pf8o_transpose_split_quant(_p(x), _p(xs) if is_fp8 else None, int(is_fp8), int(xs_layout), _p(rows), int(len(rows)), I64(K),
                                     _p(qt), _p(st), int(pow2))
    qs, ss, off = [], [], 0
    for r in rows:
        r = int(r)
        qs.append(qt[off * K:(off + r) * K].reshape(K, r))
        ss.append(st[(off // 128) * K:((off + r) // 128) * K].reshape(r // 128, K))
        off += r
    return qs, ss


def swiglu_weighted_bwd(o1, do2_s, probs):
    o1, do2_s, probs = _c(o1, np.uint16), _c(do2_s, np.uint16), _c(probs, np.float32)
    M, I2 = o1.shape
    I = I2 // 2
    do1 = np.empty((M, I2), np.uint16)
    pg = np.empty((M,), np.float32)
    o2s = np.empty((M, I), np.uint16)
    lib().pf8o_swiglu_weighted_bwd(_p(o1), _p(do2_s), _p(probs), I64(M), I64(I), _p(do1), _p(pg), _p(o2s))
    return do1, pg, o2s


def gemm_nt(a, sa, b, sb, sa_layout=0, dequant_ref=False):
    """pf8o_gemm_nt (block-scaled accumulation) or pf8o_gemm_nt_dequant_ref -> bf16 bits [M,N]."""
    a, b, sa, sb = _c(a, np.uint8), _c(b, np.uint8), _c(sa, np.float32), _c(sb, np.float32)
    M, K = a.shape
    N = b.shape[0]
    assert b.shape[1] == K and K % 128 == 0
    assert sa.shape == ((M, K // 128) if sa_layout == 0 else (K // 128, M))
    assert sb.shape == ((N + 127) // 128, K // 128)
    out = np.empty((M, N), np.uint16)
    fn = lib().pf8o_gemm_nt_dequant_ref if dequant_ref else lib().pf8o_gemm_nt
    fn(_p(a), _p(sa), int(sa_layout), _p(b), _p(sb), I64(M), I64(N), I64(K), _p(out))
    return out


def gemm_nt_1d1d_f32(a_t, sa_t, b_t, sb_t, out=None):
    a_t, b_t, sa_t, sb_t = _c(a_t, np.uint8), _c(b_t, np.uint8), _c(sa_t, np.float32), _c(sb_t, np.float32)
    Kin, M = a_t.shape
    N = b_t.shape[0]
    assert b_t.shape[1] == M and M % 128 == 0
    assert sa_t.shape == (M // 128, Kin) and sb_t.shape == (M // 128, N)
    acc = out is not None
    if out is None:
        out = np.empty((Kin, N), np.float32)
    else:
        out = _c(out, np.float32).copy()
    lib().pf8o_gemm_nt_1d1d_f32(_p(a_t), _p(sa_t), _p(b_t), _p(sb_t), I64(Kin), I64(N), I64(M), _p(out), int(acc))
    return out


def grouped_gemm_nt_contiguous(a, sa, b, sb, m_indices, sa_layout=0, out=None):
    a, b, sa, sb = _c(a, np.uint8), _c(b, np.uint8), _c(sa, np.float32), _c(sb, np.float32)
    m_indices = _c(m_indices, np.int32)
    Mtot, K = a.shape
    E, N, _ = b.shape
    assert sb.shape == (E, (N + 127) // 128, K // 128)
    out = np.zeros((Mtot, N), np.uint16) if out is None else out
    lib().pf8o_grouped_gemm_nt_contiguous(_p(a), _p(sa), int(sa_layout), _p(b), _p(sb), int(E), I64(Mtot), I64(N), I64(K),
                                          _p(m_indices), _p(out))
    return out


def grouped_gemm_nt_masked(a, sa, b, sb, masked_m, out=None):
    a, b, sa, sb = _c(a, np.uint8), _c(b, np.uint8), _c(sa, np.float32), _c(sb, np.float32)
    masked_m = _c(masked_m, np.int32)
    E, Mmax, K = a.shape
    N = b.shape[1]
    out = np.zeros((E, Mmax, N), np.uint16) if out is None else out
    lib().pf8o_grouped_gemm_nt_masked(_p(a), _p(sa), _p(b), _p(sb), int(E), I64(Mmax), I64(N), I64(K), _p(masked_m), _p(out))
    return out


# ---------------------------------------------------------------------------------------------
# block-FP8 checkpoint dequantization (numpy restatement; pinned by the reference's own known-answer
# tests, tests/coverage_test/quantization/test_coverage_hf_checkpoint_dequant.py:210-289)
# ---------------------------------------------------------------------------------------------


def ue8m0_table() -> np.ndarray:
    """quantization/checkpoint_dequant.py:93: 2^(code-127), code 255 -> inf."""
    t = np.array([2.0 ** (e - 127) for e in range(256)], dtype=np.float64)
    t[255] = np.inf
    return t.astype(np.float32)


def decode_scales(scale: np.ndarray, scale_format: str) -> np.ndarray:
    """checkpoint_dequant.py:177-183 (_decode_scales): UE8M0 codes through the table (int8 storage is
    reinterpreted as unsigned, :100-108), float formats widened to fp32; bf16 comes as uint16 bits."""
    fmt = scale_format.strip().lower()
    if fmt in ("ue8m0", "e8m0", "float8_e8m0"):
        assert scale.dtype in (np.uint8, np.int8)
        return ue8m0_table()[scale.view(np.uint8)]
    if fmt in ("bf16", "bfloat16"):
        return bf16_bits_to_f32(scale)
    return scale.astype(np.float32)


def scales_to_ue8m0(scale: np.ndarray) -> np.ndarray:
    """fp32 powers of two -> UE8M0 exponent bytes (the biased exponent field of the float).  Inverse
    of decode_scales(..., "ue8m0"), whose table follows quantization/checkpoint_dequant.py:121-131;
    the CPU tests pin it by that round trip over every finite exponent."""
    bits = np.ascontiguousarray(scale, dtype=np.float32).view(np.uint32)
    if np.any(bits & np.uint32(0x807FFFFF)):
        raise ValueError("scale is not a positive power of two")
    return (bits >> np.uint32(23)).astype(np.uint8)


def block_dequant(q: np.ndarray, scale: np.ndarray, scale_format: str, block_axes, block_shape, out: str = "f32") -> np.ndarray:
    """FP8BlockCheckpointDequantizer.dequantize (checkpoint_dequant.py:277-292): decode the e4m3 codes
    (:76-90, :111-118), expand the scale grid by repeating it block_size times along every blocked
    axis and cropping to the weight's shape (:145-176), multiply in fp32, cast.  Returns fp32 values
    or bf16 bit patterns."""
    assert q.dtype in (np.uint8, np.int8)
    vals = e4m3_decode_np(q.view(np.uint8))
    sc = decode_scales(scale, scale_format)
    if sc.ndim != vals.ndim:
        raise ValueError("Scale rank must match logical weight rank")
    axis_to_block = dict(zip([a + vals.ndim if a < 0 else a for a in block_axes], block_shape))
    expected = tuple(-(-d // axis_to_block[ax]) if ax in axis_to_block else d for ax, d in enumerate(vals.shape))
    if tuple(sc.shape) != expected:
        raise ValueError(f"Invalid scale grid shape: expected {expected}, got {tuple(sc.shape)}")
    for ax, bs in sorted(axis_to_block.items()):
        sc = np.repeat(sc, bs, axis=ax)
    sc = sc[tuple(slice(0, d) for d in vals.shape)]
    with np.errstate(invalid="ignore", over="ignore"):
        prod = (vals * sc).astype(np.float32)
    return prod if out == "f32" else f32_to_bf16_bits(prod)


# ---------------------------------------------------------------------------------------------
# moe_permute / moe_unpermute (numpy restatement).  The operators live in the paddlepaddle-gpu binary
# and the reference holds no test or fixture for them.  Pinned: the row order and content of the
# permutation and the scatter-add back, against the un-fused statement the reference keeps in plain
# tensor operations (topk_to_permuted_indices / permute_fast / unpermute_fast,
# cli/train/deepseek_v3_pretrain/moe_utils.py:57-130; tests/test_oracle_ops.py).  PARITY UNPINNED: what
# only the fused operators define -- zero rows up to a multiple of padding_alignment, the
# [T, num_experts] row map with -1 for "not routed", fp32 summation in slot order on the way back --
# taken from what the call sites rely on (moe_utils.py:141-261).
# ---------------------------------------------------------------------------------------------


def moe_permute(x, xs, routemap, probs, num_experts, tokens_per_expert, padding_alignment):
    """x: uint16 bf16 bits or uint8 e4m3 codes [T, H]; xs fp32 [T, H/128] or None."""
    T, H = x.shape
    a = padding_alignment
    padded = [(int(c) + a - 1) // a * a for c in tokens_per_expert]
    starts = np.concatenate([[0], np.cumsum(padded)]).astype(np.int64)
    mpad = int(starts[-1])
    out_x = np.zeros((mpad, H), dtype=x.dtype)
    out_p = np.zeros((mpad, 1), dtype=np.float32)
    out_s = None if xs is None else np.zeros((mpad, xs.shape[1]), dtype=np.float32)
    rowmap = np.full((T, num_experts), -1, dtype=np.int32)
    fill = np.zeros(num_experts, dtype=np.int64)
    for t in range(T):
        for e in sorted(set(int(v) for v in routemap[t] if 0 <= v < num_experts)):
            rowmap[t, e] = starts[e] + fill[e]
            fill[e] += 1
    assert (fill <= np.asarray(tokens_per_expert)).all()
    for t in range(T):
        for k in range(routemap.shape[1]):
            e = int(routemap[t, k])
            if e < 0 or e >= num_experts:
                continue
            r = rowmap[t, e]
            out_x[r] = x[t]
            if probs is not None:
                out_p[r, 0] = probs[t, k]
            if xs is not None:
                out_s[r] = xs[t]
    return out_x, rowmap, out_p, out_s


def moe_unpermute(unzipped_bits, rowmap, routemap, probs_unzipped, total_tokens, num_experts):
    T, topk = total_tokens, routemap.shape[1]
    H = unzipped_bits.shape[1]
    u = bf16_bits_to_f32(unzipped_bits)
    acc = np.zeros((T, H), dtype=np.float32)
    out_p = np.zeros((T, topk), dtype=np.float32)
    for t in range(T):
        for k in range(topk):
            e = int(routemap[t, k])
            if e < 0 or e >= num_experts or rowmap[t, e] < 0:
                continue
            acc[t] = (acc[t] + u[rowmap[t, e]]).astype(np.float32)
            if probs_unzipped is not None:
                out_p[t, k] = probs_unzipped.reshape(-1)[rowmap[t, e]]
    return f32_to_bf16_bits(acc), out_p
