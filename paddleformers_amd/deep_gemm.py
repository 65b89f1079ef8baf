"""Drop-in for the `deep_gemm` module object the reference binds at import time
(`from paddlefleet_ops import deep_gemm`, transformers/fp8_utils.py:34-44).

Same function names and argument conventions: operands are `(fp8_tensor, scale_tensor)` pairs,
the output tensor is allocated by the caller and written in place.  Everything runs through the
MFMA kernels of libpf8 on the current stream.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import torch

from . import _lib
from .functional import FP8, GatheredRows, _dev, _p, _scale_layout_of, _stream


def set_num_sms(num: int) -> None:
    """deep_gemm.set_num_sms(get_sm_num()) -- transformers/fp8_utils.py:277.  Caps the compute
    units the GEMM grids assume (0 = the whole device)."""
    _lib.lib().pf8_set_num_cus(int(num))


def get_num_sms() -> int:
    return int(_lib.lib().pf8_get_num_cus())


class FragmentMajor:
    """A quantized weight [N, K] or [E, N, K] whose bytes are stored in the order the matrix instructions consume
    them (`pf8_weight_to_fragment_major`): pass it in place of the plain e4m3 tensor of a `(b, sb)` pair and
    `fp8_gemm_nt` / `m_grouped_fp8_gemm_nt_contiguous` run the kernel that loads weight fragments straight into
    registers.  Same bytes, same scales, results equal to the plain kernels' to the matrix pipe's precision; made once per cached weight by `to_fragment_major`.
    No counterpart in the reference, whose FP8 weight cache is read by deep_gemm only."""

    __slots__ = ("data", "shape")

    def __init__(self, data: torch.Tensor, shape):
        self.data, self.shape = data, tuple(shape)

    def dim(self) -> int:
        return len(self.shape)


def fragment_major_supported(M: int, N: int, K: int) -> bool:
    """Shapes the fragment-major kernels take (whole 128-row tiles, 256-column tiles of which the last may be half new, at
    least three K blocks)."""
    return bool(_lib.lib().pf8_gemm_fm_supported(int(M), int(N), int(K)))


def to_fragment_major(w: torch.Tensor) -> FragmentMajor:
    """Fragment-major copy of an e4m3 weight [N, K] or [E, N, K] (N % 64 == 0, K % 128 == 0)."""
    _dev(w, "w")
    if w.dtype != FP8 or w.dim() not in (2, 3):
        raise ValueError("w must be float8_e4m3fn [N, K] or [E, N, K]")
    w = w if w.is_contiguous() else w.contiguous()
    E = w.shape[0] if w.dim() == 3 else 1
    N, K = w.shape[-2], w.shape[-1]
    out = torch.empty_like(w)
    _lib.call("pf8_weight_to_fragment_major", _p(w), E, N, K, _p(out), _stream())
    return FragmentMajor(out, w.shape)


def _check_pair(pair, what, gathered_ok=False) -> Tuple[torch.Tensor, torch.Tensor]:
    if not (isinstance(pair, (tuple, list)) and len(pair) == 2):
        raise ValueError(f"{what} must be a (tensor, scale) pair")
    t, s = pair
    if isinstance(t, GatheredRows):
        if not gathered_ok:
            raise ValueError(f"{what}: gathered rows are read by m_grouped_fp8_gemm_nt_contiguous only (materialize() them)")
        if s is not None:
            raise ValueError(f"{what}: gathered rows carry their own scales (pass None)")
        return t, None
    if isinstance(t, FragmentMajor):
        _dev(t.data, what)
        _dev(s, what + " scale")
        return t, s
    _dev(t, what)
    _dev(s, what + " scale")
    if t.dtype != FP8:
        raise ValueError(f"{what} must be float8_e4m3fn")
    return t, s


def _is_ue8m0(s: torch.Tensor) -> bool:
    return s.dtype == torch.uint8 or s.dtype == getattr(torch, "float8_e8m0fnu", None)


def _ue8m0_kmajor(s: torch.Tensor, rows: int, kb: int, what: str) -> torch.Tensor:
    """Exponent bytes logically [rows, K/128] -> the K-block-major [K/128, ld] storage the kernel reads
    (ld a multiple of 8).  The `.T` view of such a tensor is consumed without a copy."""
    s = s.view(torch.uint8)
    if tuple(s.shape) != (rows, kb):
        raise ValueError(f"{what} must be [{rows}, {kb}]")
    if s.stride(0) == 1 and s.stride(1) >= rows and s.stride(1) % 8 == 0 and s.data_ptr() % 8 == 0:
        return s.t()
    ld = (rows + 7) // 8 * 8
    buf = torch.empty((kb, ld), dtype=torch.uint8, device=s.device)
    buf[:, :rows].copy_(s.t())
    return buf[:, :rows]


def _decode_ue8m0(s: torch.Tensor) -> torch.Tensor:
    return torch.exp2(s.view(torch.uint8).to(torch.float32) - 127.0)


def _ue8m0_kernel_shape(M: int, N: int, K: int, experts: int = 0) -> bool:
    """Shapes the block-scaled MFMA kernel takes: 256-column tiles, the last one may be a 128-column half.
    A grouped launch with such a half tile cannot fall back to the 128-row-tile kernel on the device
    (that kernel wants whole 256-column tiles), so the choice the list header would make there is made
    here from an upper bound of the number of paired tiles (every expert with an odd block)."""
    if not (M % 128 == 0 and N % 128 == 0 and N >= 256 and K % 128 == 0 and K >= 384):
        return False
    if experts and N % 256 != 0:
        cus = int(_lib.lib().pf8_effective_num_cus())
        p_tiles = (N + 255) // 256
        rounds_pair = -(-(M // 256 + experts) * p_tiles // cus)
        rounds_128 = -(-(M // 128) * p_tiles // cus)
        return 16 * rounds_pair <= 10 * rounds_128
    return True


def fp8_gemm_nt(a, b, out: torch.Tensor, c: Optional[torch.Tensor] = None, recipe=None, compiled_dims: str = "nk"):
    """out[M, N] = a[M, K] . b[N, K]^T with block scales, fp32 accumulation.

    Default recipe (transformers/fp8_utils.py:278): a is 1x128-scaled with sa logically [M, K/128]
    (any strides; the M-contiguous `.T` view of a [K/128, M] tensor is consumed without a copy),
    b is 128x128-scaled with sb [ceil(N/128), K/128]; out is bf16.  Scales of dtype uint8 (or
    float8_e8m0fnu) are UE8M0 exponent bytes, scale = 2^(byte - 127), in the same logical shapes.
    recipe=(1, 1, 128) (transformers/fp8_utils.py:187-194): both operands 1x128-scaled along K with
    scales logically [rows, K/128]; out is fp32 and `c is out` means accumulate.
    """
    (ta, sa), (tb, sb) = _check_pair(a, "a"), _check_pair(b, "b")
    _dev(out, "out")
    M, K = ta.shape
    N, K2 = tb.shape
    if K != K2 or K % 128 != 0:
        raise ValueError("a and b must share a K that is a multiple of 128")
    if tuple(out.shape) != (M, N):
        raise ValueError(f"out must be [{M}, {N}]")
    if M == 0 or N == 0:
        return out
    fm = isinstance(tb, FragmentMajor)
    if fm and (recipe is not None or c is not None or _is_ue8m0(sa) or _is_ue8m0(sb) or not fragment_major_supported(M, N, K)
               or out.dtype != torch.bfloat16 or out.stride(-1) != 1 or out.stride(0) % 8 != 0 or out.data_ptr() % 16 != 0):
        raise ValueError("a fragment-major weight serves the default recipe with fp32 scales, M % 128 == 0, N % 128 == 0, N >= 256, K % 128 == 0, K >= 384")
    ta = ta if ta.is_contiguous() else ta.contiguous()
    if fm:
        sa, lay = _scale_layout_of(sa, M, K // 128, "a scale")
        if tuple(sb.shape) != (N // 128, K // 128) or sb.dtype != torch.float32:
            raise ValueError(f"b scale must be float32 [{N // 128}, {K // 128}]")
        _lib.call("pf8_gemm_nt_fm", _p(ta), _p(sa), lay, _p(tb.data), _p(sb.contiguous()), M, N, K, _p(out), out.stride(0), _stream())
        return out
    tb = tb if tb.is_contiguous() else tb.contiguous()
    if recipe is not None and tuple(recipe) == (1, 1, 128):
        if out.dtype != torch.float32 or not out.is_contiguous():
            raise ValueError("the (1, 1, 128) recipe writes a contiguous float32 output")
        if c is not None and c is not out and c.data_ptr() != out.data_ptr():
            raise ValueError("c must be the output tensor (in-place accumulation)")
        # scales arrive as [rows, K/128] views of [K/128, rows] storage; the kernel wants the latter
        sa_k = sa.t() if sa.t().is_contiguous() else sa.t().contiguous()
        sb_k = sb.t() if sb.t().is_contiguous() else sb.t().contiguous()
        if tuple(sa_k.shape) != (K // 128, M) or tuple(sb_k.shape) != (K // 128, N):
            raise ValueError("scales must be [rows, K/128]")
        _lib.call("pf8_gemm_nt_1d1d_f32", _p(ta), _p(sa_k), _p(tb), _p(sb_k), M, N, K, _p(out), int(c is not None), _stream())
        return out
    if recipe is not None:
        raise ValueError(f"unsupported recipe {recipe!r}")
    if c is not None:
        raise ValueError("accumulation needs recipe=(1, 1, 128)")
    if out.dtype != torch.bfloat16 or out.stride(-1) != 1:
        raise ValueError("out must be bfloat16 with a unit inner stride")
    if _is_ue8m0(sa) != _is_ue8m0(sb):
        raise ValueError("UE8M0 scales must be given for both operands or for neither")
    if _is_ue8m0(sa):
        # power-of-two scales as exponent bytes (`use_ue8m0`, transformers/configuration_utils.py:454-459):
        # the block-scaled MFMA kernel where its tile shape fits, else the fp32-scale kernel on decoded scales
        if tuple(sb.shape) != ((N + 127) // 128, K // 128):
            raise ValueError(f"b scale must be [{(N + 127) // 128}, {K // 128}]")
        if _ue8m0_kernel_shape(M, N, K) and out.stride(0) % 8 == 0 and out.data_ptr() % 16 == 0:
            sa_k = _ue8m0_kmajor(sa, M, K // 128, "a scale")
            sb_k = sb.view(torch.uint8).contiguous()
            _lib.call("pf8_gemm_nt_ue8m0", _p(ta), _p(sa_k), sa_k.stride(0), _p(tb), _p(sb_k), M, N, K, _p(out), out.stride(0), _stream())
            return out
        sa, sb = _decode_ue8m0(sa), _decode_ue8m0(sb)
    sa, lay = _scale_layout_of(sa, M, K // 128, "a scale")
    if tuple(sb.shape) != ((N + 127) // 128, K // 128) or sb.dtype != torch.float32:
        raise ValueError(f"b scale must be float32 [{(N + 127) // 128}, {K // 128}]")
    sb = sb if sb.is_contiguous() else sb.contiguous()
    _lib.call("pf8_gemm_nt", _p(ta), _p(sa), lay, _p(tb), _p(sb), M, N, K, _p(out), out.stride(0), _stream())
    return out


def build_group_items(m_indices: torch.Tensor) -> torch.Tensor:
    """Work-item list of the UE8M0 grouped GEMM for one m_indices (int32 [Mtot], Mtot a multiple of 128):
    pass it as `items=` to every m_grouped_fp8_gemm_nt_contiguous call that shares the m_indices
    (up+gate, down, dgrad).  No counterpart in the reference API; without it each call builds its own."""
    _dev(m_indices, "m_indices")
    if m_indices.dtype != torch.int32 or m_indices.numel() % 128 != 0:
        raise ValueError("m_indices must be int32 with a multiple of 128 entries")
    m_indices = m_indices if m_indices.is_contiguous() else m_indices.contiguous()
    items = torch.empty(4 + 4 * (m_indices.numel() // 128), dtype=torch.int32, device=m_indices.device)
    _lib.call("pf8_grouped_items_build", _p(m_indices), m_indices.numel(), _p(items), _stream())
    return items


def m_grouped_fp8_gemm_nt_contiguous(a, b, out: torch.Tensor, m_indices: torch.Tensor, items: Optional[torch.Tensor] = None):
    """Grouped GEMM over rows sorted by expert: row m uses b[m_indices[m]].

    transformers/fp8_utils.py:949-954: a [Mtot, K] + sa [Mtot, K/128] (any strides), b [E, N, K] +
    sb [E, N/128, K/128], m_indices int32 [Mtot]; every expert segment is a multiple of 128 rows.
    a may be `(GatheredRows, None)` with a fragment-major b: the rows are then read from the tokens through the source
    map, with the result the copied rows would give, to the bit.
    `items` (optional, UE8M0 scales only): the list build_group_items made for this m_indices.
    """
    (ta, sa), (tb, sb) = _check_pair(a, "a", gathered_ok=True), _check_pair(b, "b")
    _dev(out, "out")
    _dev(m_indices, "m_indices")
    Mtot, K = ta.shape
    if tb.dim() != 3:
        raise ValueError("b must be [E, N, K]")
    E, N, K2 = tb.shape
    if K != K2 or K % 128 != 0:
        raise ValueError("a and b must share a K that is a multiple of 128")
    if Mtot % 128 != 0:
        raise ValueError("the row count must be a multiple of 128 (expert segments are padded to 128)")
    if tuple(out.shape) != (Mtot, N) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous bfloat16 [{Mtot}, {N}] tensor")
    if m_indices.dtype != torch.int32 or m_indices.numel() != Mtot:
        raise ValueError("m_indices must be int32 with one entry per row")
    if Mtot == 0 or N == 0:
        return out
    ta = ta.contiguous()
    m_indices = m_indices if m_indices.is_contiguous() else m_indices.contiguous()
    if isinstance(ta, GatheredRows):
        if not isinstance(tb, FragmentMajor) or _is_ue8m0(sb) or not fragment_major_supported(Mtot, N, K):
            raise ValueError("gathered rows go with a fragment-major weight and fp32 scales (materialize() them for the other kernels)")
        if tuple(sb.shape) != (E, N // 128, K // 128) or sb.dtype != torch.float32:
            raise ValueError(f"b scale must be float32 [{E}, {N // 128}, {K // 128}]")
        T = ta.tokens.shape[0]
        if ta.tokens.dtype != FP8:
            raise ValueError("gathered bfloat16 tokens have to be quantized first (GatheredRows.quantize)")
        if T == 0 or T * K >= 2 ** 31 or ta.src_row.data_ptr() % 16:
            raise ValueError("gathered rows: the token matrix must be non-empty and below 2 GiB, the source map 16-byte aligned")
        rs, lay = _scale_layout_of(ta.row_scales(), Mtot, K // 128, "row scales")
        _lib.call("pf8_grouped_gemm_nt_contiguous_fm_gather", _p(ta.tokens), T, _p(ta.src_row), _p(rs), lay, _p(tb.data), _p(sb.contiguous()),
                  E, Mtot, N, K, _p(m_indices), _p(out), _stream())
        return out
    if isinstance(tb, FragmentMajor):
        if _is_ue8m0(sa) or _is_ue8m0(sb) or not fragment_major_supported(Mtot, N, K):
            raise ValueError("a fragment-major weight serves fp32 scales, Mtot % 128 == 0, N % 128 == 0, N >= 256, K % 128 == 0, K >= 384")
        sa, lay = _scale_layout_of(sa, Mtot, K // 128, "a scale")
        if tuple(sb.shape) != (E, N // 128, K // 128) or sb.dtype != torch.float32:
            raise ValueError(f"b scale must be float32 [{E}, {N // 128}, {K // 128}]")
        _lib.call("pf8_grouped_gemm_nt_contiguous_fm", _p(ta), _p(sa), lay, _p(tb.data), _p(sb.contiguous()), E, Mtot, N, K,
                  _p(m_indices), _p(out), _stream())
        return out
    tb = tb if tb.is_contiguous() else tb.contiguous()
    if _is_ue8m0(sa) != _is_ue8m0(sb):
        raise ValueError("UE8M0 scales must be given for both operands or for neither")
    if _is_ue8m0(sa):
        if tuple(sb.shape) != (E, (N + 127) // 128, K // 128):
            raise ValueError(f"b scale must be [{E}, {(N + 127) // 128}, {K // 128}]")
        if _ue8m0_kernel_shape(Mtot, N, K, E):
            sa_k = _ue8m0_kmajor(sa, Mtot, K // 128, "a scale")
            sb_k = sb.view(torch.uint8).contiguous()
            if items is None:
                items = build_group_items(m_indices)
            elif items.dtype != torch.int32 or items.numel() != 4 + 4 * (Mtot // 128) or not items.is_contiguous():
                raise ValueError("items must come from build_group_items for this m_indices")
            _lib.call("pf8_grouped_gemm_nt_contiguous_ue8m0", _p(ta), _p(sa_k), sa_k.stride(0), _p(tb), _p(sb_k), E, Mtot, N, K,
                      _p(m_indices), _p(items), _p(out), _stream())
            return out
        sa, sb = _decode_ue8m0(sa), _decode_ue8m0(sb)
    sa, lay = _scale_layout_of(sa, Mtot, K // 128, "a scale")
    if tuple(sb.shape) != (E, (N + 127) // 128, K // 128) or sb.dtype != torch.float32:
        raise ValueError(f"b scale must be float32 [{E}, {(N + 127) // 128}, {K // 128}]")
    sb = sb if sb.is_contiguous() else sb.contiguous()
    _lib.call("pf8_grouped_gemm_nt_contiguous", _p(ta), _p(sa), lay, _p(tb), _p(sb), E, Mtot, N, K, _p(m_indices), _p(out), _stream())
    return out


def swiglu_quant_fusable(Mtot: int, N: int, K: int, a_scale: Optional[torch.Tensor] = None,
                         b_scale: Optional[torch.Tensor] = None) -> bool:
    """Shapes and scale kinds m_grouped_fp8_gemm_nt_contiguous_swiglu_quant takes: fp32 scales, whole 128-row and
    128-column tiles of both halves, at least three K blocks."""
    if (a_scale is not None and _is_ue8m0(a_scale)) or (b_scale is not None and _is_ue8m0(b_scale)):
        return False
    return Mtot > 0 and Mtot % 128 == 0 and N % 256 == 0 and N > 0 and K % 128 == 0 and K >= 384


def m_grouped_fp8_gemm_nt_contiguous_swiglu_quant(a, b, m_indices: torch.Tensor, probs: Optional[torch.Tensor] = None,
                                                  using_pow2_scaling: bool = False, out: Optional[torch.Tensor] = None):
    """The up+gate grouped GEMM of the MoE MLP with fused_weighted_swiglu_act_quant in its epilogue: one launch for
    transformers/fp8_utils.py:949-954 followed by :981-987.  a [Mtot, K] + sa, b [E, 2I, K] (gate rows, then up rows)
    + sb [E, 2I/128, K/128], fp32 scales; probs fp32 [Mtot] (or [Mtot, 1]) or None.  Returns (q [Mtot, I] e4m3,
    s [Mtot, I/128] fp32), bit-identical to m_grouped_fp8_gemm_nt_contiguous + fused_weighted_swiglu_act_quant;
    `out` (bf16 [Mtot, 2I], optional) also receives the GEMM result o1.  No counterpart of its own in the reference."""
    (ta, sa), (tb, sb) = _check_pair(a, "a"), _check_pair(b, "b")
    _dev(m_indices, "m_indices")
    Mtot, K = ta.shape
    if tb.dim() != 3:
        raise ValueError("b must be [E, 2I, K]")
    E, N, K2 = tb.shape
    if K != K2 or not swiglu_quant_fusable(Mtot, N, K, sa, sb):
        raise ValueError("shape or scale kind outside the fused kernel: Mtot % 128 == 0, 2I % 256 == 0, K % 128 == 0, K >= 384, fp32 scales")
    I = N // 2
    if m_indices.dtype != torch.int32 or m_indices.numel() != Mtot:
        raise ValueError("m_indices must be int32 with one entry per row")
    if out is not None:
        _dev(out, "out")
        if tuple(out.shape) != (Mtot, N) or out.dtype != torch.bfloat16 or not out.is_contiguous():
            raise ValueError(f"out must be a contiguous bfloat16 [{Mtot}, {N}] tensor")
    if probs is not None:
        _dev(probs, "probs")
        probs = probs.reshape(-1)
        if probs.numel() != Mtot:
            raise ValueError("probs must have one entry per row")
        probs = probs.float().contiguous()
    ta = ta if ta.is_contiguous() else ta.contiguous()
    tb = tb if tb.is_contiguous() else tb.contiguous()
    m_indices = m_indices if m_indices.is_contiguous() else m_indices.contiguous()
    sa, lay = _scale_layout_of(sa, Mtot, K // 128, "a scale")
    if tuple(sb.shape) != (E, N // 128, K // 128) or sb.dtype != torch.float32:
        raise ValueError(f"b scale must be float32 [{E}, {N // 128}, {K // 128}]")
    sb = sb if sb.is_contiguous() else sb.contiguous()
    q = torch.empty((Mtot, I), dtype=FP8, device=ta.device)
    s = torch.empty((I // 128, Mtot), dtype=torch.float32, device=ta.device)        # handed back as its transpose (see the quantizer)
    _lib.call("pf8_grouped_gemm_swiglu_quant_nt_contiguous", _p(ta), _p(sa), lay, _p(tb), _p(sb), E, Mtot, I, K, _p(m_indices),
              _p(probs), _p(out), _p(q), _p(s), int(bool(using_pow2_scaling)) | 2, _stream())
    return q, s.t()


def m_grouped_fp8_gemm_nt_masked(a, b, out: torch.Tensor, masked_m: torch.Tensor, expected_m: int):
    """Grouped GEMM with a fixed capacity per expert.

    ernie token_dispatcher/fp8_utils.py:227-233: a [E, Mmax, K] + sa [E, Mmax, K/128], b [E, N, K] +
    sb [E, N/128, K/128], masked_m int32 [E]; rows at or beyond masked_m[e] are not written.
    """
    (ta, sa), (tb, sb) = _check_pair(a, "a"), _check_pair(b, "b")
    _dev(out, "out")
    _dev(masked_m, "masked_m")
    if ta.dim() != 3 or tb.dim() != 3:
        raise ValueError("a must be [E, Mmax, K] and b [E, N, K]")
    E, Mmax, K = ta.shape
    E2, N, K2 = tb.shape
    if E != E2 or K != K2 or K % 128 != 0:
        raise ValueError("a and b must agree on E and on a K that is a multiple of 128")
    if tuple(out.shape) != (E, Mmax, N) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous bfloat16 [{E}, {Mmax}, {N}] tensor")
    if masked_m.dtype != torch.int32 or masked_m.numel() != E:
        raise ValueError("masked_m must be int32 [E]")
    if E == 0 or Mmax == 0 or N == 0:
        return out
    ta, tb = ta.contiguous(), tb.contiguous()
    if tuple(sa.shape) != (E, Mmax, K // 128) or tuple(sb.shape) != (E, (N + 127) // 128, K // 128):
        raise ValueError("scale shapes must be [E, Mmax, K/128] and [E, N/128, K/128]")
    sa, sb = sa.contiguous(), sb.contiguous()
    _lib.call("pf8_grouped_gemm_nt_masked", _p(ta), _p(sa), _p(tb), _p(sb), E, Mmax, N, K, _p(masked_m.contiguous()), int(expected_m),
              _p(out), _stream())
    return out


# names the reference aliases when it falls back to paddle.incubate.fp8.deep_gemm (fp8_utils.py:42-44)
gemm_fp8_fp8_bf16_nt = fp8_gemm_nt
m_grouped_gemm_fp8_fp8_bf16_nt_contiguous = m_grouped_fp8_gemm_nt_contiguous
m_grouped_gemm_fp8_fp8_bf16_nt_masked = m_grouped_fp8_gemm_nt_masked
