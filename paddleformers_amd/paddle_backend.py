"""Paddle-side binding of libpf8.so: the file a PaddleFormers maintainer adds as paddleformers/utils/pf8_backend.py.

install() puts a `paddlefleet_ops` module with a `deep_gemm` attribute into sys.modules (what
paddleformers/transformers/fp8_utils.py:34-44 imports) and assigns the quantizer operators onto
paddle.incubate.nn.functional, all through the C ABI of include/pf8.h.  Paddle tensors go in as raw device pointers,
outputs are allocated with paddle.empty where the reference allocates them, the stream is Paddle's current stream.
Importing this module needs Paddle; nothing else in this package imports it.
"""
import ctypes, sys, types
import paddle

_lib = ctypes.CDLL("libpf8.so")
_vp, _i64, _i32, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
_lib.pf8_last_error.restype = ctypes.c_char_p
FP8, F32, BF16 = paddle.float8_e4m3fn, paddle.float32, paddle.bfloat16

def _p(t):      return None if t is None else _vp(t.data_ptr())
def _stream():  return _vp(paddle.device.current_stream().stream_base.raw_stream)
def _b(flag):   return _i32(int(bool(flag)))
def _dense(t):  return t if t.is_contiguous() else t.contiguous()
def _call(name, *args):
    rc = getattr(_lib, name)(*args)
    if rc:
        msg = _lib.pf8_last_error().decode()
        raise (ValueError if rc == -1 else RuntimeError)(f"{name}: {msg}")

def _scale_layout(s, rows, blocks):
    """A logical [rows, blocks] fp32 scale tensor -> (tensor, scale_layout): 0 = row-major,
    1 = the `.T` view of a [blocks, rows] tensor (what output_scale_transpose=True + `.T` gives)."""
    assert list(s.shape) == [rows, blocks] and s.dtype == F32
    if s.is_contiguous():            return s, 0
    if list(s.strides) == [1, rows]: return s, 1
    return s.contiguous(), 0

# ---- paddle.incubate.nn.functional.* ---------------------------------------------------------

def fp8_quant_blockwise(x, quant_method="1x128", input_transpose=False, output_scale_transpose=False,
                        return_transpose_only=False, using_pow2_scale=False, **unused):
    x2 = _dense(x.reshape([-1, x.shape[-1]]))
    M, K = x2.shape
    lay, pow2 = int(bool(output_scale_transpose)), _b(using_pow2_scale)
    if quant_method == "1x128" and not input_transpose:
        q = paddle.empty([M, K], dtype=FP8)
        s = paddle.empty([K // 128, M] if lay else [M, K // 128], dtype=F32)
        _call("pf8_quant_1x128", _p(x2), _i64(M), _i64(K), _i64(K), _p(q), _p(s), _i32(lay), pow2, _stream())
        return q.reshape(x.shape), s
    if quant_method == "1x128":                       # row-scaled copy + column-scaled transposed copy
        q = s = None
        if not return_transpose_only:
            q = paddle.empty([M, K], dtype=FP8)
            s = paddle.empty([K // 128, M] if lay else [M, K // 128], dtype=F32)
        q_t = paddle.empty([K, M], dtype=FP8)
        s_t = paddle.empty([M // 128, K] if lay else [K, M // 128], dtype=F32)
        _call("pf8_quant_transpose", _p(x2), _i64(M), _i64(K), _p(q), _p(s), _p(q_t), _p(s_t), _i32(lay), pow2, _stream())
        return (q_t, s_t) if return_transpose_only else (q, s, q_t, s_t)
    if quant_method == "128x128":
        q = s = q_t = s_t = None
        if not return_transpose_only:
            q = paddle.empty([M, K], dtype=FP8)
            s = paddle.empty([M // 128, K // 128], dtype=F32)
        if input_transpose:
            q_t = paddle.empty([K, M], dtype=FP8)
            s_t = paddle.empty([K // 128, M // 128], dtype=F32)
        _call("pf8_quant_128x128", _p(x2), _i64(M), _i64(K), _p(q), _p(s), _p(q_t), _p(s_t), pow2, _stream())
        if return_transpose_only: return q_t, s_t
        return (q, s, q_t, s_t) if input_transpose else (q, s)
    raise ValueError(f"unsupported quant_method {quant_method!r}")

def fused_stack_transpose_quant(weight_list, transpose=False):
    ws = [_dense(w) for w in weight_list]             # keep the contiguous copies alive over the call
    E, (R, C) = len(ws), ws[0].shape
    rows, cols = (E * C, R) if transpose else (E * R, C)
    q = paddle.empty([rows, cols], dtype=FP8)
    s = paddle.empty([rows // 128, cols // 128], dtype=F32)
    ptrs = (_vp * E)(*[w.data_ptr() for w in ws])
    _call("pf8_stack_transpose_quant", ptrs, _i32(E), _i64(R), _i64(C), _b(transpose), _p(q), _p(s), _i32(0), _stream())
    return q, s

def fused_weighted_swiglu_act_quant(o1, probs=None, using_pow2_scaling=False):
    o1 = _dense(o1)
    M, I = o1.shape[0], o1.shape[1] // 2
    if probs is not None:
        probs = _dense(probs.reshape([-1]).astype(F32))
    q = paddle.empty([M, I], dtype=FP8)
    s = paddle.empty([M, I // 128], dtype=F32)
    _call("pf8_swiglu_weighted_quant", _p(o1), _p(probs), _i64(M), _i64(I), _p(q), _p(s), None, _i32(0),
          _b(using_pow2_scaling), _stream())
    return q, s

def fused_transpose_split_quant(x, scale, tokens_per_expert, pow_2_scales=False):
    x = _dense(x)
    Mtot, K = x.shape
    rows = [int(t) for t in tokens_per_expert]
    assert sum(rows) == Mtot and len(rows) <= 256     # more experts: call once per 256 (functional.py does)
    is_fp8, lay = x.dtype == FP8, 0
    if is_fp8:
        scale, lay = _scale_layout(scale, Mtot, K // 128)
    q_t = paddle.empty([K * Mtot], dtype=FP8)         # one packed buffer, the per-expert tensors are views of it
    s_t = paddle.empty([(Mtot // 128) * K], dtype=F32)
    arr = (_i64 * len(rows))(*rows)
    _call("pf8_transpose_split_quant", _p(x), _p(scale) if is_fp8 else None, _b(is_fp8), _i32(lay), arr, _i32(len(rows)),
          _i64(K), _p(q_t), _p(s_t), _b(pow_2_scales), _stream())
    qs, ss, off = [], [], 0
    for r in rows:
        qs.append(q_t[off * K:(off + r) * K].reshape([K, r]))
        ss.append(s_t[(off // 128) * K:((off + r) // 128) * K].reshape([r // 128, K]))
        off += r
    return qs, ss

def fused_act_dequant(q, scale):
    q = _dense(q)
    M, K = q.shape
    scale, lay = _scale_layout(scale, M, K // 128)
    out = paddle.empty([M, K], dtype=BF16)
    _call("pf8_act_dequant", _p(q), _p(scale), _i32(lay), _i64(M), _i64(K), _p(out), _stream())
    return out

def fused_swiglu_weighted_bwd(o1, do2_s, probs):
    o1, do2_s = _dense(o1), _dense(do2_s)
    M, I = o1.shape[0], o1.shape[1] // 2
    probs = _dense(probs.reshape([-1]).astype(F32))
    do1 = paddle.empty([M, 2 * I], dtype=BF16)
    probs_grad = paddle.empty([M], dtype=F32)
    o2_s = paddle.empty([M, I], dtype=BF16)
    _call("pf8_swiglu_weighted_bwd", _p(o1), _p(do2_s), _p(probs), _i64(M), _i64(I), _p(do1), _p(probs_grad), _p(o2_s), _stream())
    return do1, probs_grad, o2_s

def fp8_gemm_blockwise(a, a_decode_scale, b, b_decode_scale, out_dtype=F32, out=None, accumulate=False,
                       use_split_accumulator=True, is_a_1d_scaled=True, is_b_1d_scaled=True):
    if not (is_a_1d_scaled and is_b_1d_scaled):
        raise ValueError("only the 1x128-by-1x128 scaled form is implemented")
    a, b = _dense(a), _dense(b)
    (Ka, M), Nb = a.shape, b.shape[0]
    sa, sb = _dense(a_decode_scale), _dense(b_decode_scale)          # [M/128, Ka], [M/128, Nb]
    if out is None:
        assert not accumulate and out_dtype == F32
        out = paddle.empty([Ka, Nb], dtype=F32)
    _call("pf8_gemm_nt_1d1d_f32", _p(a), _p(sa), _p(b), _p(sb), _i64(Ka), _i64(Nb), _i64(M), _p(out), _b(accumulate), _stream())
    return out

# ---- paddlefleet_ops.deep_gemm ---------------------------------------------------------------

deep_gemm = types.ModuleType("deep_gemm")

def _is_ue8m0(s): return s.dtype == paddle.uint8

def _ue8m0_kmajor(s, rows, kb):
    """Exponent bytes logically [rows, K/128] -> (tensor, ldsa) in the [K/128, ldsa] storage the kernel reads."""
    if list(s.strides)[0] == 1 and s.strides[1] >= rows and s.strides[1] % 8 == 0 and s.data_ptr() % 8 == 0:
        return s, s.strides[1]                        # the `.T` view of a [K/128, ld] tensor: no copy
    ld = (rows + 7) // 8 * 8
    buf = paddle.empty([kb, ld], dtype=paddle.uint8)
    buf[:, :rows] = s.t()
    return buf, ld

def _decode_ue8m0(s): return 2.0 ** (s.astype(F32) - 127.0)

def _ue8m0_shape_ok(M, N, K):
    return M % 128 == 0 and N % 256 == 0 and K % 128 == 0 and K >= 384

def _fp8_gemm_nt(a, b, out, c=None, recipe=None, compiled_dims="nk"):
    (ta, sa), (tb, sb) = a, b
    ta, tb = _dense(ta), _dense(tb)
    (M, K), N = ta.shape, tb.shape[0]
    if M == 0 or N == 0:
        return out
    if recipe is not None:                            # (1, 1, 128): both 1x128-scaled, fp32 out, `c is out` accumulates
        assert tuple(recipe) == (1, 1, 128) and out.dtype == F32
        sa_k, sb_k = _dense(sa.t()), _dense(sb.t())   # callers pass `.t()` of [K/128, rows]: no copy
        _call("pf8_gemm_nt_1d1d_f32", _p(ta), _p(sa_k), _p(tb), _p(sb_k), _i64(M), _i64(N), _i64(K), _p(out),
              _b(c is not None), _stream())
        return out
    if _is_ue8m0(sa):
        if _ue8m0_shape_ok(M, N, K) and out.strides[0] % 8 == 0:
            sa_k, ld = _ue8m0_kmajor(sa, M, K // 128)
            _call("pf8_gemm_nt_ue8m0", _p(ta), _p(sa_k), _i64(ld), _p(tb), _p(_dense(sb)), _i64(M), _i64(N), _i64(K),
                  _p(out), _i64(out.strides[0]), _stream())
            return out
        sa, sb = _decode_ue8m0(sa), _decode_ue8m0(sb)
    sa, lay = _scale_layout(sa, M, K // 128)
    _call("pf8_gemm_nt", _p(ta), _p(sa), _i32(lay), _p(tb), _p(_dense(sb)), _i64(M), _i64(N), _i64(K), _p(out),
          _i64(out.strides[0]), _stream())
    return out

def _build_group_items(m_indices):
    items = paddle.empty([4 + 4 * (m_indices.shape[0] // 128)], dtype=paddle.int32)
    _call("pf8_grouped_items_build", _p(m_indices), _i64(m_indices.shape[0]), _p(items), _stream())
    return items

def _grouped_contiguous(a, b, out, m_indices, items=None):
    (ta, sa), (tb, sb) = a, b
    ta, tb, m_indices = _dense(ta), _dense(tb), _dense(m_indices)
    (Mtot, K), (E, N, _) = ta.shape, tb.shape
    if Mtot == 0 or N == 0:
        return out
    if _is_ue8m0(sa):
        if _ue8m0_shape_ok(Mtot, N, K):
            sa_k, ld = _ue8m0_kmajor(sa, Mtot, K // 128)
            if items is None:                         # reusable by every GEMM of the step that shares m_indices
                items = _build_group_items(m_indices)
            _call("pf8_grouped_gemm_nt_contiguous_ue8m0", _p(ta), _p(sa_k), _i64(ld), _p(tb), _p(_dense(sb)), _i32(E),
                  _i64(Mtot), _i64(N), _i64(K), _p(m_indices), _p(items), _p(out), _stream())
            return out
        sa, sb = _decode_ue8m0(sa), _decode_ue8m0(sb)
    sa, lay = _scale_layout(sa, Mtot, K // 128)
    _call("pf8_grouped_gemm_nt_contiguous", _p(ta), _p(sa), _i32(lay), _p(tb), _p(_dense(sb)), _i32(E), _i64(Mtot),
          _i64(N), _i64(K), _p(m_indices), _p(out), _stream())
    return out

def _grouped_masked(a, b, out, masked_m, expected_m):
    (ta, sa), (tb, sb) = a, b
    ta, tb = _dense(ta), _dense(tb)
    (E, Mmax, K), N = ta.shape, tb.shape[1]
    if E == 0 or Mmax == 0 or N == 0:
        return out
    _call("pf8_grouped_gemm_nt_masked", _p(ta), _p(_dense(sa)), _p(tb), _p(_dense(sb)), _i32(E), _i64(Mmax), _i64(N),
          _i64(K), _p(_dense(masked_m.astype(paddle.int32))), _i32(int(expected_m)), _p(out), _stream())
    return out

def _set_num_sms(n): _lib.pf8_set_num_cus(_i32(int(n)))
def _get_num_sms():  return int(_lib.pf8_get_num_cus())

deep_gemm.fp8_gemm_nt = _fp8_gemm_nt
deep_gemm.m_grouped_fp8_gemm_nt_contiguous = _grouped_contiguous
deep_gemm.m_grouped_fp8_gemm_nt_masked = _grouped_masked
deep_gemm.build_group_items = _build_group_items
deep_gemm.set_num_sms = _set_num_sms
deep_gemm.get_num_sms = _get_num_sms

def install():
    ops = types.ModuleType("paddlefleet_ops")
    ops.deep_gemm = deep_gemm
    sys.modules["paddlefleet_ops"] = ops              # picked up by fp8_utils.py:34
    F = paddle.incubate.nn.functional
    for fn in (fp8_quant_blockwise, fused_stack_transpose_quant, fused_weighted_swiglu_act_quant,
               fused_transpose_split_quant, fused_act_dequant, fused_swiglu_weighted_bwd, fp8_gemm_blockwise):
        setattr(F, fn.__name__, fn)
