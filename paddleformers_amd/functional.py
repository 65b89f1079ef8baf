"""Drop-in replacements for the `paddle.incubate.nn.functional` FP8 operators the reference calls.

Same names, keyword arguments, output shapes and scale conventions as the call sites in
paddleformers/transformers/fp8_utils.py; tensors are device tensors (torch-ROCm here: bf16 =
torch.bfloat16, e4m3 = torch.float8_e4m3fn, scales fp32) and every function launches a libpf8
kernel on the current stream.  There is no CPU path: a CPU tensor raises.
"""
from __future__ import annotations

import collections.abc
import ctypes as C
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib

FP8 = torch.float8_e4m3fn


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t: torch.Tensor, what: str) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{what} must be a tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{what} must live on the GPU: libpf8 has no CPU path")
    return t


def _p(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _as2d(x: torch.Tensor) -> torch.Tensor:
    return x.reshape(-1, x.shape[-1])


class GatheredRows:
    """The expert-sorted, padded rows `moe_permute` would write, not copied: row r is row src_row[r] of `tokens`;
    src_row[r] < 0 is a row of zeros.  `tokens` is float8_e4m3fn [T, H] with `scale` fp32 [T, H/128] (dispatched FP8
    tokens, quantized gradients), or bfloat16 [T, H] with `scale` None (gradient tokens before quantization).
    What `moe_permute(..., do_gather=False)` returns in place of the copied rows; `m_grouped_fp8_gemm_nt_contiguous` (e4m3
    tokens, on a fragment-major weight) and `fused_transpose_split_quant` take it where they take the copied rows and read
    the tokens through the map, with bit-identical results.  A slice `g[a:b]` is the same tokens behind a slice of the map."""

    __slots__ = ("tokens", "scale", "src_row", "_row_scale")

    def __init__(self, tokens: torch.Tensor, scale: Optional[torch.Tensor], src_row: torch.Tensor):
        if tokens.dim() != 2 or not tokens.is_contiguous() or tokens.dtype not in (FP8, torch.bfloat16):
            raise ValueError("tokens must be a contiguous float8_e4m3fn or bfloat16 [T, H] tensor")
        if tokens.dtype == FP8:
            if scale is None or scale.dtype != torch.float32 or tuple(scale.shape) != (tokens.shape[0], tokens.shape[1] // 128) \
                    or not scale.is_contiguous():
                raise ValueError("float8 tokens come with a contiguous float32 [T, H/128] scale tensor")
        elif scale is not None:
            raise ValueError("bfloat16 tokens carry no scale")
        if src_row.dtype != torch.int32 or src_row.dim() != 1:
            raise ValueError("src_row must be int32 [rows]")
        self.tokens, self.scale, self.src_row = tokens, scale, src_row
        self._row_scale = None

    def row_scales(self) -> torch.Tensor:
        """The scales of the expert-sorted rows, fp32 logical [rows, H/128] stored [H/128, rows] (what the GEMMs read
        without a copy), zero on rows of zeros: gathered from the token scales on first use (4 bytes per row and block
        against the 128 bytes they scale) and kept."""
        if self.tokens.dtype != FP8:
            raise ValueError("bfloat16 tokens carry no scales (quantize() first)")
        if self._row_scale is None:
            rows, KB = self.src_row.shape[0], self.scale.shape[1]
            src = self.src_row if self.src_row.is_contiguous() else self.src_row.contiguous()
            out = torch.empty((KB, rows), dtype=torch.float32, device=self.device)
            if rows and KB:
                _lib.call("pf8_gather_row_scales", _p(self.scale), self.tokens.shape[0], KB, _p(src), rows, _p(out), 1, _stream())
            self._row_scale = out.t()
        return self._row_scale

    @property
    def shape(self):
        return torch.Size((self.src_row.shape[0], self.tokens.shape[1]))

    @property
    def device(self):
        return self.tokens.device

    @property
    def dtype(self):
        return self.tokens.dtype

    def dim(self) -> int:
        return 2

    def __getitem__(self, sl):
        if not isinstance(sl, slice) or sl.step not in (None, 1):
            raise TypeError("only contiguous row slices of gathered rows can be taken")
        return GatheredRows(self.tokens, self.scale, self.src_row[sl])       # (its row scales are gathered anew: they are stored per slice)

    def contiguous(self):
        if self.src_row.is_contiguous():
            return self
        g = GatheredRows(self.tokens, self.scale, self.src_row.contiguous())
        g._row_scale = self._row_scale
        return g

    def quantize(self, using_pow2_scale: bool = False) -> "GatheredRows":
        """bfloat16 tokens -> the same rows behind their 1x128-quantized tokens.  The rule is per row, so quantizing the T
        tokens once gives every copy the bytes and scales that quantizing the copied rows would (and a row of zeros stays
        one)."""
        if self.tokens.dtype == FP8:
            return self
        q, s = fp8_quant_blockwise(self.tokens, quant_method="1x128", using_pow2_scale=using_pow2_scale)
        return GatheredRows(q, s, self.src_row)

    def materialize(self):
        """The copy, for a consumer that cannot read through the map: (rows e4m3 [rows, H], scales fp32 [rows, H/128]) for
        float8 tokens, rows bfloat16 [rows, H] for bfloat16 tokens."""
        live = self.src_row >= 0
        idx = self.src_row.clamp(min=0).long()
        if self.tokens.dtype == FP8:
            rows = self.tokens.view(torch.uint8)[idx] * live[:, None].to(torch.uint8)
            return rows.view(FP8), self.scale[idx] * live[:, None].to(torch.float32)
        return torch.where(live[:, None], self.tokens[idx], torch.zeros((), dtype=torch.bfloat16, device=self.device))


def _scale_layout_of(s: torch.Tensor, rows: int, blocks: int, what: str, allow_ue8m0: bool = False) -> Tuple[torch.Tensor, int]:
    """A logical [rows, blocks] scale tensor -> (tensor, layout flag) without copying when its
    memory is either row-major (0) or blocks-major, i.e. a transposed view of [blocks, rows] (1);
    UE8M0 exponent bytes (uint8, where the caller takes them) are layout 2, blocks-major."""
    if tuple(s.shape) != (rows, blocks):
        raise ValueError(f"{what} must have shape [{rows}, {blocks}], got {list(s.shape)}")
    if s.dtype == torch.uint8 and allow_ue8m0:          # UE8M0 bytes: blocks-major only
        return (s if s.stride() == (1, rows) else s.t().contiguous().t()), 2
    if s.dtype != torch.float32:
        raise ValueError(f"{what} must be float32")
    if s.is_contiguous():
        return s, 0
    if s.stride() == (1, rows):
        return s, 1
    return s.contiguous(), 0


# ---------------------------------------------------------------------------------------------
# fp8_quant_blockwise
# ---------------------------------------------------------------------------------------------


def fp8_quant_blockwise(
    x: torch.Tensor,
    quant_method: str = "1x128",
    input_transpose: bool = False,
    output_scale_transpose: bool = False,
    return_transpose_only: bool = False,
    using_pow2_scale: bool = False,
    ue8m0_scale: bool = False,
):
    """Block-wise e4m3 quantization, scale = amax/448 per tile.

    Mirrors the keyword use at transformers/fp8_utils.py:112-131 (128x128 weights) and
    :158-173, :262-268 (1x128 activations).  Returns (q, s), (q, s, q_t, s_t) when
    input_transpose, or (q_t, s_t) when also return_transpose_only.
    Scale shapes: 1x128 -> [M, K/128], or [K/128, M] with output_scale_transpose (transposed copy:
    [K, M/128] / [M/128, K]); 128x128 -> [R/128, C/128] (transposed copy [C/128, R/128]).
    ue8m0_scale (1x128 without input_transpose, power-of-two scales): the scales come back as UE8M0 exponent bytes
    (uint8, scale = 2^(byte - 127)) of the same logical shape, stored [K/128, M] -- the form the block-scaled GEMMs of
    `use_ue8m0` (transformers/configuration_utils.py:454-459) read, written by the quantizer itself.
    """
    _dev(x, "x")
    if x.dtype != torch.bfloat16:
        raise ValueError("fp8_quant_blockwise expects a bfloat16 tensor")
    if return_transpose_only and not input_transpose:
        raise ValueError("return_transpose_only requires input_transpose=True")
    x2 = _as2d(x)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    M, K = x2.shape
    pow2 = int(bool(using_pow2_scale))
    dev = x.device
    if quant_method == "1x128":
        if K % 128 != 0:
            raise ValueError(f"last dimension must be divisible by 128, got {K}")
        lay = 1 if output_scale_transpose else 0
        if ue8m0_scale:
            if input_transpose or not pow2:
                raise ValueError("ue8m0_scale goes with using_pow2_scale=True and input_transpose=False")
            q = torch.empty((M, K), dtype=FP8, device=dev)
            s = torch.empty((K // 128, M), dtype=torch.uint8, device=dev)
            _lib.call("pf8_quant_1x128", _p(x2), M, K, K, _p(q), _p(s), 2, 1, _stream())
            return q.reshape(x.shape), (s if output_scale_transpose else s.t())
        if not input_transpose:
            q = torch.empty((M, K), dtype=FP8, device=dev)
            s = torch.empty((K // 128, M) if lay else (M, K // 128), dtype=torch.float32, device=dev)
            _lib.call("pf8_quant_1x128", _p(x2), M, K, K, _p(q), _p(s), lay, pow2, _stream())
            return q.reshape(x.shape), s
        if M % 128 != 0:
            raise ValueError(f"input_transpose=True needs the row count to be a multiple of 128, got {M}")
        q = s = None
        if not return_transpose_only:
            q = torch.empty((M, K), dtype=FP8, device=dev)
            s = torch.empty((K // 128, M) if lay else (M, K // 128), dtype=torch.float32, device=dev)
        q_t = torch.empty((K, M), dtype=FP8, device=dev)
        s_t = torch.empty((M // 128, K) if lay else (K, M // 128), dtype=torch.float32, device=dev)
        _lib.call("pf8_quant_transpose", _p(x2), M, K, _p(q), _p(s), _p(q_t), _p(s_t), lay, pow2, _stream())
        if return_transpose_only:
            return q_t, s_t
        return q, s, q_t, s_t
    if quant_method == "128x128":
        if M % 128 != 0 or K % 128 != 0:
            raise ValueError(f"128x128 quantization needs both dimensions divisible by 128, got [{M}, {K}]")
        if output_scale_transpose:
            raise ValueError("128x128 quantization has no output_scale_transpose layout")
        q = s = q_t = s_t = None
        if not return_transpose_only:
            q = torch.empty((M, K), dtype=FP8, device=dev)
            s = torch.empty((M // 128, K // 128), dtype=torch.float32, device=dev)
        if input_transpose:
            q_t = torch.empty((K, M), dtype=FP8, device=dev)
            s_t = torch.empty((K // 128, M // 128), dtype=torch.float32, device=dev)
        _lib.call("pf8_quant_128x128", _p(x2), M, K, _p(q), _p(s), _p(q_t), _p(s_t), pow2, _stream())
        if return_transpose_only:
            return q_t, s_t
        if input_transpose:
            return q, s, q_t, s_t
        return q, s
    raise ValueError(f"unsupported quant_method {quant_method!r} (expected '1x128' or '128x128')")


# ---------------------------------------------------------------------------------------------
# fused_stack_transpose_quant
# ---------------------------------------------------------------------------------------------


def fused_stack_transpose_quant(weight_list: Sequence[torch.Tensor], transpose: bool = False, using_pow2_scale: bool = False):
    """Stack E bf16 [R, C] weights, optionally transposing each, and quantize in 128x128 tiles.

    transformers/fp8_utils.py:101; un-fused equivalent ernie token_dispatcher/fp8_utils.py:276-287.
    Returns q [E*R, C] (or [E*C, R] with transpose) and s [E*R/128, C/128] (or [E*C/128, R/128]).
    """
    if len(weight_list) == 0:
        raise ValueError("weight_list is empty")
    R, Cc = weight_list[0].shape
    ws = []
    for w in weight_list:
        _dev(w, "weight")
        if w.dtype != torch.bfloat16 or tuple(w.shape) != (R, Cc):
            raise ValueError("all weights must be bfloat16 with the same 2-D shape")
        ws.append(w if w.is_contiguous() else w.contiguous())
    if R % 128 != 0 or Cc % 128 != 0:
        raise ValueError(f"weight dimensions must be divisible by 128, got [{R}, {Cc}]")
    E = len(ws)
    dev = ws[0].device
    if transpose:
        q = torch.empty((E * Cc, R), dtype=FP8, device=dev)
        s = torch.empty((E * Cc // 128, R // 128), dtype=torch.float32, device=dev)
    else:
        q = torch.empty((E * R, Cc), dtype=FP8, device=dev)
        s = torch.empty((E * R // 128, Cc // 128), dtype=torch.float32, device=dev)
    ptrs = (C.c_void_p * E)(*[w.data_ptr() for w in ws])
    _lib.call("pf8_stack_transpose_quant", ptrs, E, R, Cc, int(bool(transpose)), _p(q), _p(s), int(bool(using_pow2_scale)), _stream())
    return q, s


def fused_stack_quant_both(weight_list: Sequence[torch.Tensor], using_pow2_scale: bool = False, fragment_major=False):
    """Both orientations of `fused_stack_transpose_quant` from one read of the weights.

    Returns (q, s, q_t, s_t) equal to `fused_stack_transpose_quant(ws, False)` +
    `fused_stack_transpose_quant(ws, True)`: the pair DeepseekV2MoE.fp8_quant_weight builds with two
    calls when quant_transpose is None (cli/train/deepseek_v3_pretrain/modeling.py:521-534).
    fragment_major: True, or a pair of flags for (q, q_t): the same pass also writes the fragment-major copies
    the `*_fm` GEMMs read, and the result is (q, s, q_t, s_t, q_fm, q_t_fm) with None where none was asked for;
    each equals `pf8_weight_to_fragment_major` of its plain tensor to the byte.
    """
    if len(weight_list) == 0:
        raise ValueError("weight_list is empty")
    R, Cc = weight_list[0].shape
    ws = []
    for w in weight_list:
        _dev(w, "weight")
        if w.dtype != torch.bfloat16 or tuple(w.shape) != (R, Cc):
            raise ValueError("all weights must be bfloat16 with the same 2-D shape")
        ws.append(w if w.is_contiguous() else w.contiguous())
    if R % 128 != 0 or Cc % 128 != 0:
        raise ValueError(f"weight dimensions must be divisible by 128, got [{R}, {Cc}]")
    E = len(ws)
    dev = ws[0].device
    q = torch.empty((E * R, Cc), dtype=FP8, device=dev)
    s = torch.empty((E * R // 128, Cc // 128), dtype=torch.float32, device=dev)
    qt = torch.empty((E * Cc, R), dtype=FP8, device=dev)
    st = torch.empty((E * Cc // 128, R // 128), dtype=torch.float32, device=dev)
    ptrs = (C.c_void_p * E)(*[w.data_ptr() for w in ws])
    want_fm = (bool(fragment_major),) * 2 if isinstance(fragment_major, bool) else tuple(bool(f) for f in fragment_major)
    if any(want_fm):
        q_fm = torch.empty_like(q) if want_fm[0] else None
        qt_fm = torch.empty_like(qt) if want_fm[1] else None
        _lib.call("pf8_stack_quant_both_fm", ptrs, E, R, Cc, _p(q), _p(s), _p(qt), _p(st), _p(q_fm), _p(qt_fm),
                  int(bool(using_pow2_scale)), _stream())
        return q, s, qt, st, q_fm, qt_fm
    _lib.call("pf8_stack_quant_both", ptrs, E, R, Cc, _p(q), _p(s), _p(qt), _p(st), int(bool(using_pow2_scale)), _stream())
    return (q, s, qt, st, None, None) if not isinstance(fragment_major, bool) else (q, s, qt, st)


# ---------------------------------------------------------------------------------------------
# fused_weighted_swiglu_act_quant
# ---------------------------------------------------------------------------------------------


def fused_weighted_swiglu_act_quant(o1: torch.Tensor, probs: Optional[torch.Tensor] = None, using_pow2_scaling: bool = False,
                                    return_o2: bool = False, ue8m0_scale: bool = False):
    """quant_1x128( bf16( bf16(swiglu(o1)) * probs ) ) in one pass.

    transformers/fp8_utils.py:984-986; un-fused equivalent ernie token_dispatcher/fp8_utils.py:996-1004.
    o1 bf16 [M, 2I] with the gate in the first half; probs fp32 [M] (or [M, 1]) or None.
    Returns (q [M, I], s [M, I/128]); with return_o2 also the bf16 activations before quantization.
    ue8m0_scale (with using_pow2_scaling): s is UE8M0 exponent bytes, uint8 [M, I/128] stored [I/128, M].
    """
    _dev(o1, "o1")
    if o1.dtype != torch.bfloat16 or o1.dim() != 2:
        raise ValueError("o1 must be a 2-D bfloat16 tensor")
    if not o1.is_contiguous():
        o1 = o1.contiguous()
    M, I2 = o1.shape
    if I2 % 256 != 0:
        raise ValueError(f"o1 last dimension must be a multiple of 256, got {I2}")
    I = I2 // 2
    if probs is not None:
        _dev(probs, "probs")
        probs = probs.reshape(-1)
        if probs.numel() != M:
            raise ValueError("probs must have one entry per row of o1")
        if probs.dtype != torch.float32:
            probs = probs.float()
        probs = probs.contiguous()
    q = torch.empty((M, I), dtype=FP8, device=o1.device)
    o2 = torch.empty((M, I), dtype=torch.bfloat16, device=o1.device) if return_o2 else None
    if ue8m0_scale:
        if not using_pow2_scaling:
            raise ValueError("ue8m0_scale goes with using_pow2_scaling=True")
        s = torch.empty((I // 128, M), dtype=torch.uint8, device=o1.device)
        _lib.call("pf8_swiglu_weighted_quant", _p(o1), _p(probs), M, I, _p(q), _p(s), _p(o2), 2, 1, _stream())
        s = s.t()
    else:
        # stored [I/128, M] and handed back as its transpose: the same [M, I/128] tensor to every consumer, in the layout the
        # grouped GEMM that follows reads fastest (one 256-byte piece per 64 rows and K block instead of 64 separate words)
        s = torch.empty((I // 128, M), dtype=torch.float32, device=o1.device)
        _lib.call("pf8_swiglu_weighted_quant", _p(o1), _p(probs), M, I, _p(q), _p(s), _p(o2), 1, int(bool(using_pow2_scaling)), _stream())
        s = s.t()
    return (q, s, o2) if return_o2 else (q, s)


# ---------------------------------------------------------------------------------------------
# fused_transpose_split_quant
# ---------------------------------------------------------------------------------------------


class _PackedExperts(collections.abc.Sequence):
    """The per-expert tensors fused_transpose_split_quant returns (one q_t [K, M_e] or s_t [M_e/128, K] per expert, empty
    tensors for experts without rows), as views of the one packed buffer the kernel wrote.  The views are made when an
    entry is asked for: with 128 experts, slicing 256 of them up front costs more host time than the kernel runs.
    `grouped_wgrad` takes the buffer as it is."""

    def __init__(self, buf: torch.Tensor, rows: List[int], K: int, scales: bool):
        self.buf, self.rows, self.K, self.scales = buf, rows, K, scales
        self._start = None
        self._views = {}

    def __len__(self):
        return len(self.rows)

    def __add__(self, other):          # list + list, as code written for the reference's lists may do
        return list(self) + list(other)

    def __radd__(self, other):
        return list(other) + list(self)

    def __getitem__(self, i):
        if isinstance(i, slice):
            return [self[j] for j in range(*i.indices(len(self.rows)))]
        if i < 0:
            i += len(self.rows)
        if not 0 <= i < len(self.rows):
            raise IndexError(i)
        v = self._views.get(i)
        if v is None:
            if self._start is None:
                self._start = [0]
                for r in self.rows:
                    self._start.append(self._start[-1] + r)
            off, r, K = self._start[i], self.rows[i], self.K
            if self.scales:
                v = self.buf[(off // 128) * K:((off + r) // 128) * K].view(r // 128, K)
            else:
                v = self.buf[off * K:(off + r) * K].view(K, r)
            self._views[i] = v
        return v


def fused_transpose_split_quant(x: torch.Tensor, scale: Optional[torch.Tensor], tokens_per_expert: Sequence[int],
                                pow_2_scales: bool = False) -> Tuple[List[torch.Tensor], List[torch.Tensor]]:
    """Per-expert split along rows -> transpose -> 1x128 quantization along the token axis.

    transformers/fp8_utils.py:1096-1100; un-fused equivalent ernie token_dispatcher/fp8_utils.py:1199-1210.
    x is bf16 [sum(M_e), K], or e4m3 with its [sum(M_e), K/128] scales (dequantized to bf16 first).
    Returns lists with one q_t [K, M_e] and one s_t [M_e/128, K] per expert (empty tensors for
    experts without rows).
    """
    gathered = x if isinstance(x, GatheredRows) else None
    if gathered is not None:
        if scale is not None:
            raise ValueError("gathered rows carry their own scales")
        x = gathered.tokens
    _dev(x, "x")
    if x.dim() != 2:
        raise ValueError("x must be 2-D")
    if not x.is_contiguous():
        x = x.contiguous()
    Mtot, K = x.shape if gathered is None else gathered.shape
    rows = [int(t) for t in tokens_per_expert]
    if sum(rows) != Mtot:
        raise ValueError(f"tokens_per_expert sums to {sum(rows)} but x has {Mtot} rows")
    if any(r % 128 != 0 or r < 0 for r in rows):
        raise ValueError("every tokens_per_expert entry must be a non-negative multiple of 128")
    if K % 128 != 0:
        raise ValueError(f"last dimension must be divisible by 128, got {K}")
    if gathered is not None:
        return _transpose_split_quant_gathered(gathered, rows, pow_2_scales)
    is_fp8 = x.dtype == FP8
    xs_layout = 0
    if is_fp8:
        if scale is None:
            raise ValueError("an e4m3 input needs its scale tensor")
        _dev(scale, "scale")
        scale, xs_layout = _scale_layout_of(scale, Mtot, K // 128, "scale", allow_ue8m0=True)
    elif x.dtype != torch.bfloat16:
        raise ValueError("x must be bfloat16 or float8_e4m3fn")
    E = len(rows)
    q_t = torch.empty((K * Mtot,), dtype=FP8, device=x.device)
    s_t = torch.empty(((Mtot // 128) * K,), dtype=torch.float32, device=x.device)
    for e0 in range(0, E, 256):
        chunk = rows[e0:e0 + 256]
        off = sum(rows[:e0])
        n = sum(chunk)
        arr = (C.c_int64 * len(chunk))(*chunk)
        xs_ptr, lay, keep = None, 0, None
        if is_fp8:
            if n == Mtot:
                xs_ptr, lay = _p(scale), xs_layout
            else:
                # more than 256 experts: hand each chunk its own slice of the scales (row-major fp32, blocks-major bytes)
                if xs_layout == 2:
                    keep = scale[off:off + n].t().contiguous()
                    xs_ptr, lay = _p(keep), 2
                else:
                    keep = scale[off:off + n].contiguous()
                    xs_ptr, lay = _p(keep), 0
        xp = C.c_void_p(x.data_ptr() + off * K * x.element_size())
        qp = C.c_void_p(q_t.data_ptr() + off * K)
        sp = C.c_void_p(s_t.data_ptr() + (off // 128) * K * 4)
        _lib.call("pf8_transpose_split_quant", xp, xs_ptr, int(is_fp8), lay, arr, len(chunk), K, qp, sp, int(bool(pow_2_scales)), _stream())
    return _PackedExperts(q_t, rows, K, False), _PackedExperts(s_t, rows, K, True)


def _transpose_split_quant_gathered(g: GatheredRows, rows: List[int], pow_2_scales: bool):
    """fused_transpose_split_quant of rows that are read through their source map (rows already checked)."""
    Mtot, K = g.shape
    T = g.tokens.shape[0]
    if T == 0 and Mtot:
        raise ValueError("gathered rows need a non-empty token matrix")
    src = g.src_row if g.src_row.is_contiguous() else g.src_row.contiguous()
    q_t = torch.empty((K * Mtot,), dtype=FP8, device=g.device)
    s_t = torch.empty(((Mtot // 128) * K,), dtype=torch.float32, device=g.device)
    for e0 in range(0, len(rows), 256):
        chunk = rows[e0:e0 + 256]
        off = sum(rows[:e0])
        if sum(chunk) == 0:
            continue
        arr = (C.c_int64 * len(chunk))(*chunk)
        _lib.call("pf8_transpose_split_quant_gather", _p(g.tokens), _p(g.scale), int(g.tokens.dtype == FP8), 0, T,
                  C.c_void_p(src.data_ptr() + off * 4), arr, len(chunk), K,
                  C.c_void_p(q_t.data_ptr() + off * K), C.c_void_p(s_t.data_ptr() + (off // 128) * K * 4), int(bool(pow_2_scales)), _stream())
    return _PackedExperts(q_t, rows, K, False), _PackedExperts(s_t, rows, K, True)


def quant_and_transpose_split(x: torch.Tensor, tokens_per_expert: Sequence[int], using_pow2_scale: bool = False,
                              pow_2_scales: bool = True, ue8m0_scale: bool = False):
    """fp8_quant_blockwise(x, quant_method="1x128", output_scale_transpose=True, using_pow2_scale=...) and
    fused_transpose_split_quant(x, None, tokens_per_expert, pow_2_scales) from ONE read of x: the two
    quantizations the MoE node's backward applies to the same gradient (transformers/fp8_utils.py:1030-1036
    with :1115, :1073-1079 with :1168).  Returns (q [M,K], s [K/128,M], q_t list, s_t list), each
    bit-identical to the separate calls' outputs.  At most 256 experts.
    ue8m0_scale (with using_pow2_scale): s comes back as UE8M0 exponent bytes, uint8 [K/128, M]."""
    _dev(x, "x")
    if x.dim() != 2 or x.dtype != torch.bfloat16:
        raise ValueError("x must be a 2-D bfloat16 tensor")
    if not x.is_contiguous():
        x = x.contiguous()
    Mtot, K = x.shape
    rows = [int(t) for t in tokens_per_expert]
    if sum(rows) != Mtot:
        raise ValueError(f"tokens_per_expert sums to {sum(rows)} but x has {Mtot} rows")
    if any(r % 128 != 0 or r < 0 for r in rows):
        raise ValueError("every tokens_per_expert entry must be a non-negative multiple of 128")
    if K % 128 != 0:
        raise ValueError(f"last dimension must be divisible by 128, got {K}")
    if len(rows) > 256:
        raise ValueError("at most 256 experts")
    if ue8m0_scale and not using_pow2_scale:
        raise ValueError("ue8m0_scale goes with using_pow2_scale=True")
    q = torch.empty((Mtot, K), dtype=FP8, device=x.device)
    s = torch.empty((K // 128, Mtot), dtype=torch.uint8 if ue8m0_scale else torch.float32, device=x.device)
    q_t = torch.empty((K * Mtot,), dtype=FP8, device=x.device)
    s_t = torch.empty(((Mtot // 128) * K,), dtype=torch.float32, device=x.device)
    if Mtot and K:
        arr = (C.c_int64 * len(rows))(*rows)
        _lib.call("pf8_quant_and_transpose_split", _p(x), arr, len(rows), K, _p(q), _p(s), 2 if ue8m0_scale else int(bool(using_pow2_scale)),
                  _p(q_t), _p(s_t), int(bool(pow_2_scales)), _stream())
    return q, s, _PackedExperts(q_t, rows, K, False), _PackedExperts(s_t, rows, K, True)


# ---------------------------------------------------------------------------------------------
# dequantizers
# ---------------------------------------------------------------------------------------------


def scales_to_ue8m0(scale: torch.Tensor, check: bool = True) -> torch.Tensor:
    """fp32 power-of-two scales (what the quantizers emit with using_pow2_scale=True) -> UE8M0
    exponent bytes of the same shape and strides order, scale = 2^(byte - 127): the scale format
    `use_ue8m0` hands to deep_gemm (transformers/configuration_utils.py:454-459).  With `check` the
    call synchronizes and raises if a scale is not a positive finite power of two."""
    _dev(scale, "scale")
    if scale.dtype == torch.uint8:            # already exponent bytes (a quantizer wrote them)
        return scale
    if scale.dtype != torch.float32:
        raise ValueError("scale must be float32")
    dense = scale if scale.is_contiguous() or (scale.dim() == 2 and scale.t().is_contiguous()) else scale.contiguous()
    out = torch.empty_like(dense, dtype=torch.uint8)      # preserves the strides of a dense tensor
    if out.stride() != dense.stride():
        dense = dense.contiguous()
        out = torch.empty_like(dense, dtype=torch.uint8)
    bad = torch.zeros(1, dtype=torch.int32, device=scale.device) if check else None
    _lib.call("pf8_scales_to_ue8m0", _p(dense), dense.numel(), _p(out), _p(bad), _stream())
    if check and int(bad.item()) != 0:
        raise ValueError(f"{int(bad.item())} scales are not positive powers of two")
    return out


def fused_act_dequant(q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """1x128 dequantization to bf16: bf16(float(q) * s).  transformers/fp8_utils.py:136-138, :779."""
    _dev(q, "q")
    _dev(scale, "scale")
    if q.dtype != FP8 or q.dim() != 2:
        raise ValueError("q must be a 2-D float8_e4m3fn tensor")
    if not q.is_contiguous():
        q = q.contiguous()
    M, K = q.shape
    if K % 128 != 0:
        raise ValueError(f"last dimension must be divisible by 128, got {K}")
    scale, lay = _scale_layout_of(scale, M, K // 128, "scale")
    out = torch.empty((M, K), dtype=torch.bfloat16, device=q.device)
    _lib.call("pf8_act_dequant", _p(q), _p(scale), lay, M, K, _p(out), _stream())
    return out


def weight_dequant(q: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """128x128 dequantization to bf16.  cli/train/deepseek_v3_pretrain/kernel.py:100-118 (same
    asserts: contiguous, 2-D); quantization/checkpoint_dequant.py:277-292 for ragged edges."""
    _dev(q, "x")
    _dev(s, "s")
    assert q.is_contiguous() and s.is_contiguous(), "Input tensors must be contiguous"
    assert q.dim() == 2 and s.dim() == 2, "Input tensors must have 2 dimensions"
    if block_size != 128:
        raise ValueError("only block_size=128 is supported")
    if q.dtype not in (FP8, torch.uint8, torch.int8):
        raise ValueError("x must hold e4m3 codes (float8_e4m3fn, uint8 or int8 storage)")
    R, Cc = q.shape
    if tuple(s.shape) != ((R + 127) // 128, (Cc + 127) // 128) or s.dtype != torch.float32:
        raise ValueError("s must be float32 [ceil(R/128), ceil(C/128)]")
    out = torch.empty((R, Cc), dtype=torch.bfloat16, device=q.device)
    _lib.call("pf8_weight_dequant", _p(q), _p(s), R, Cc, _p(out), _stream())
    return out


# ---------------------------------------------------------------------------------------------
# fused_swiglu_weighted_bwd
# ---------------------------------------------------------------------------------------------


def fused_swiglu_weighted_bwd(o1: torch.Tensor, do2_s: torch.Tensor, probs: torch.Tensor):
    """SwiGLU backward with per-row probs.  transformers/fp8_utils.py:1050; un-fused equivalent
    ernie token_dispatcher/fp8_utils.py:1088-1092.  Returns (do1 [M,2I] bf16, probs_grad [M] fp32,
    o2_s [M,I] bf16)."""
    for t, n in ((o1, "o1"), (do2_s, "do2_s"), (probs, "probs")):
        _dev(t, n)
    if o1.dtype != torch.bfloat16 or do2_s.dtype != torch.bfloat16:
        raise ValueError("o1 and do2_s must be bfloat16")
    o1 = o1.contiguous()
    do2_s = do2_s.contiguous()
    M, I2 = o1.shape
    I = I2 // 2
    if tuple(do2_s.shape) != (M, I):
        raise ValueError(f"do2_s must be [{M}, {I}]")
    if I % 8 != 0:
        raise ValueError("I must be a multiple of 8")
    probs = probs.reshape(-1).float().contiguous()
    if probs.numel() != M:
        raise ValueError("probs must have one entry per row")
    do1 = torch.empty((M, I2), dtype=torch.bfloat16, device=o1.device)
    pg = torch.empty((M,), dtype=torch.float32, device=o1.device)
    o2s = torch.empty((M, I), dtype=torch.bfloat16, device=o1.device)
    _lib.call("pf8_swiglu_weighted_bwd", _p(o1), _p(do2_s), _p(probs), M, I, _p(do1), _p(pg), _p(o2s), _stream())
    return do1, pg, o2s


def swiglu_weighted_bwd_quant(o1: torch.Tensor, do2_s: torch.Tensor, probs: torch.Tensor, tokens_per_expert: Sequence[int],
                              using_pow2_scale: bool = False, pow_2_scales: bool = True, ue8m0_scale: bool = False,
                              output_scale_transpose: bool = True):
    """fused_swiglu_weighted_bwd(o1, do2_s, probs) followed by quant_and_transpose_split(do1, tokens_per_expert,
    using_pow2_scale, pow_2_scales, ue8m0_scale) and fused_transpose_split_quant(o2_s, None, tokens_per_expert,
    pow_2_scales) (transformers/fp8_utils.py:1049-1052, then :1073-1079, :1168 and :1115), from one read of o1 and do2_s:
    the bf16 do1 and o2_s are never written.  Returns (do1_q [M,2I], do1_s [2I/128,M], do1_q_t list, do1_s_t list,
    o2s_q_t list, o2s_s_t list, probs_grad [M]); the quantized forms are bit-identical to the separate calls',
    probs_grad agrees with theirs to the rounding of a sum taken in another order.  At most 256 experts.
    output_scale_transpose=False: do1_s comes back [M, 2I/128], as fp8_quant_blockwise(..., output_scale_transpose=False)
    stores it (not with ue8m0_scale)."""
    for t, n in ((o1, "o1"), (do2_s, "do2_s"), (probs, "probs")):
        _dev(t, n)
    if o1.dim() != 2 or do2_s.dim() != 2 or o1.dtype != torch.bfloat16 or do2_s.dtype != torch.bfloat16:
        raise ValueError("o1 and do2_s must be 2-D bfloat16 tensors")
    o1 = o1.contiguous()
    do2_s = do2_s.contiguous()
    M, I2 = o1.shape
    I = I2 // 2
    if I2 % 2 != 0 or tuple(do2_s.shape) != (M, I):
        raise ValueError(f"do2_s must be [{M}, {I2 // 2}] for o1 [{M}, {I2}]")
    if I % 128 != 0:
        raise ValueError(f"I must be divisible by 128, got {I}")
    rows = [int(t) for t in tokens_per_expert]
    if sum(rows) != M:
        raise ValueError(f"tokens_per_expert sums to {sum(rows)} but o1 has {M} rows")
    if any(r % 128 != 0 or r < 0 for r in rows):
        raise ValueError("every tokens_per_expert entry must be a non-negative multiple of 128")
    if len(rows) > 256:
        raise ValueError("at most 256 experts")
    if ue8m0_scale and not using_pow2_scale:
        raise ValueError("ue8m0_scale goes with using_pow2_scale=True")
    if ue8m0_scale and not output_scale_transpose:
        raise ValueError("ue8m0_scale bytes are stored [2I/128, M] (output_scale_transpose=True)")
    probs = probs.reshape(-1).float().contiguous()
    if probs.numel() != M:
        raise ValueError("probs must have one entry per row")
    if probs.data_ptr() % 16:
        probs = probs.clone()
    dev = o1.device
    q = torch.empty((M, I2), dtype=FP8, device=dev)
    s = torch.empty((I2 // 128, M) if output_scale_transpose else (M, I2 // 128), dtype=torch.uint8 if ue8m0_scale else torch.float32, device=dev)
    q_t = torch.empty((I2 * M,), dtype=FP8, device=dev)
    s_t = torch.empty(((M // 128) * I2,), dtype=torch.float32, device=dev)
    oq_t = torch.empty((I * M,), dtype=FP8, device=dev)
    os_t = torch.empty(((M // 128) * I,), dtype=torch.float32, device=dev)
    pg = torch.empty((M,), dtype=torch.float32, device=dev)
    if M and I:
        part = torch.empty((I // 128, M), dtype=torch.float32, device=dev)
        arr = (C.c_int64 * len(rows))(*rows)
        _lib.call("pf8_swiglu_weighted_bwd_quant", _p(o1), _p(do2_s), _p(probs), arr, len(rows), I, _p(q), _p(s),
                  int(bool(output_scale_transpose)), 2 if ue8m0_scale else int(bool(using_pow2_scale)), _p(q_t), _p(s_t), _p(oq_t), _p(os_t), int(bool(pow_2_scales)),
                  _p(pg), _p(part), _stream())
    else:
        pg.zero_()
    return (q, s, _PackedExperts(q_t, rows, I2, False), _PackedExperts(s_t, rows, I2, True),
            _PackedExperts(oq_t, rows, I, False), _PackedExperts(os_t, rows, I, True), pg)


# ---------------------------------------------------------------------------------------------
# fp8_gemm_blockwise (weight-gradient GEMM)
# ---------------------------------------------------------------------------------------------


def fp8_gemm_blockwise(a, a_decode_scale, b, b_decode_scale, out_dtype=torch.float32, out=None, accumulate=False,
                       use_split_accumulator=True, is_a_1d_scaled=True, is_b_1d_scaled=True, scales_pow2=False):
    """y[Ka, Nb] (+)= a[Ka, M] . b[Nb, M]^T with both operands 1x128-scaled along M.

    transformers/fp8_utils.py:203-214 (kitchen_gemm): a_decode_scale [M/128, Ka], b_decode_scale
    [M/128, Nb]; fp32 output; accumulate adds into `out`.  scales_pow2 (not in the reference's
    signature): the caller vouches that every scale is a power of two, as
    fused_transpose_split_quant(..., pow_2_scales=True) makes them; the scales then go into the
    block-scaled MFMA.  Other scales would lose their mantissa unnoticed.
    """
    if not (is_a_1d_scaled and is_b_1d_scaled):
        raise ValueError("only the 1x128-by-1x128 scaled form is implemented (is_a_1d_scaled = is_b_1d_scaled = True)")
    for t, n in ((a, "a"), (b, "b"), (a_decode_scale, "a_decode_scale"), (b_decode_scale, "b_decode_scale")):
        _dev(t, n)
    if a.dtype != FP8 or b.dtype != FP8:
        raise ValueError("a and b must be float8_e4m3fn")
    a, b = a.contiguous(), b.contiguous()
    Ka, M = a.shape
    Nb, M2 = b.shape
    if M != M2 or M % 128 != 0:
        raise ValueError("a and b must share a reduction length that is a multiple of 128")
    sa = a_decode_scale.contiguous()
    sb = b_decode_scale.contiguous()
    if tuple(sa.shape) != (M // 128, Ka) or tuple(sb.shape) != (M // 128, Nb):
        raise ValueError("decode scales must be [M/128, rows]")
    if out is None:
        if accumulate:
            raise ValueError("accumulate=True needs out")
        if out_dtype != torch.float32:
            raise ValueError("the weight-gradient GEMM produces float32")
        out = torch.empty((Ka, Nb), dtype=torch.float32, device=a.device)
    else:
        if out.dtype != torch.float32 or tuple(out.shape) != (Ka, Nb) or not out.is_contiguous():
            raise ValueError("out must be a contiguous float32 [Ka, Nb] tensor")
    _lib.call("pf8_gemm_nt_1d1d_f32_pow2" if scales_pow2 else "pf8_gemm_nt_1d1d_f32", _p(a), _p(sa), _p(b), _p(sb), Ka, Nb, M, _p(out),
              int(bool(accumulate)), _stream())
    return out


def grouped_wgrad(a_t_list, sa_t_list, b_t_list, sb_t_list, out: torch.Tensor, accumulate: bool = True, scales_pow2: bool = False):
    """All experts' weight gradients in one launch: out[e] (+)= a_t[e] . b_t[e]^T.

    Replaces the per-expert Python loops of transformers/fp8_utils.py:1117-1129 and :1170-1182.
    The lists must be the outputs of fused_transpose_split_quant (views of one packed buffer);
    scales_pow2 says they were made with pow_2_scales=True (see fp8_gemm_blockwise).
    """
    E = len(a_t_list)
    packed = all(isinstance(l, _PackedExperts) for l in (a_t_list, sa_t_list, b_t_list, sb_t_list))
    if packed:
        # the quantizer's own result objects: the packing is known, no view has to be made
        rows = list(a_t_list.rows)
        Kin, N = a_t_list.K, b_t_list.K
        if list(b_t_list.rows) != rows or list(sa_t_list.rows) != rows or list(sb_t_list.rows) != rows or \
                sa_t_list.K != Kin or sb_t_list.K != N or a_t_list.scales or b_t_list.scales or not sa_t_list.scales or not sb_t_list.scales:
            raise ValueError("operands do not belong together (rows per expert, widths or roles differ)")
    else:
        rows = [int(t.shape[1]) for t in a_t_list]
        Kin = int(a_t_list[0].shape[0])
        N = int(b_t_list[0].shape[0])
    if tuple(out.shape) != (E, Kin, N) or out.dtype != torch.float32 or not out.is_contiguous():
        raise ValueError("out must be a contiguous float32 [E, Kin, N] tensor")

    def base(lst):
        if packed:
            return _p(lst.buf)
        t0 = lst[0]
        st = t0.untyped_storage()
        p = st.data_ptr() + t0.storage_offset() * t0.element_size()
        # verify the packing: each tensor must start where the previous one ends
        exp = p
        for t in lst:
            if t.numel() and t.data_ptr() != exp:
                raise ValueError("operands are not the packed outputs of fused_transpose_split_quant")
            exp += t.numel() * t.element_size()
        return C.c_void_p(p)

    arr = (C.c_int64 * E)(*rows)
    _lib.call("pf8_grouped_wgrad_pow2" if scales_pow2 else "pf8_grouped_wgrad", base(a_t_list), base(sa_t_list), base(b_t_list),
              base(sb_t_list), arr, E, Kin, N, _p(out), int(bool(accumulate)), _stream())
    return out


def swiglu(x: torch.Tensor, y: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16 SwiGLU with the kernel's arithmetic: silu(x[:, :I]) * x[:, I:].  transformers/fp8_utils.py:23-29."""
    if y is not None:
        x = torch.cat([x, y], dim=-1)
    _dev(x, "x")
    x2 = _as2d(x).contiguous()
    M, I2 = x2.shape
    I = I2 // 2
    if I % 128 != 0:
        raise ValueError("swiglu needs a half width that is a multiple of 128")
    q = torch.empty((M, I), dtype=FP8, device=x.device)
    s = torch.empty((M, I // 128), dtype=torch.float32, device=x.device)
    o2 = torch.empty((M, I), dtype=torch.bfloat16, device=x.device)
    _lib.call("pf8_swiglu_weighted_quant", _p(x2), None, M, I, _p(q), _p(s), _p(o2), 0, 0, _stream())
    return o2.reshape(*x.shape[:-1], I)


# ---------------------------------------------------------------------------------------------
# swiglu_grad, fused_rms_norm_ext(+grad): the remaining operators of the dense FP8 MLP backward
# ---------------------------------------------------------------------------------------------


def swiglu_grad(o1: torch.Tensor, y, do2: torch.Tensor):
    """paddle._C_ops.swiglu_grad(o1, None, do2) as the dense MLP backward calls it
    (transformers/fp8_utils.py:407): gradient of swiglu(o1) with the two halves packed in o1.
    Returns (do1, None).  Runs the weighted kernel with unit probabilities (bf16(do2 * 1) == do2)."""
    if y is not None:
        raise ValueError("swiglu_grad supports the packed form only (y must be None)")
    o2d = _as2d(o1)
    ones = torch.ones((o2d.shape[0],), dtype=torch.float32, device=o1.device)
    do1, _, _ = fused_swiglu_weighted_bwd(o2d, _as2d(do2), ones)
    return do1.reshape(o1.shape), None


def fused_rms_norm_ext(x: torch.Tensor, norm_weight: torch.Tensor, epsilon: float):
    """paddle.incubate.nn.functional.fused_rms_norm_ext(x, norm_w, eps) -> (y, invvar)
    (transformers/fp8_utils.py:472, 522, 691).  x bf16 [..., H], norm_weight bf16 [H];
    y = bf16(x * invvar * w) with invvar fp32 [rows] = 1/sqrt(mean(x^2) + eps)."""
    _dev(x, "x")
    _dev(norm_weight, "norm_weight")
    if x.dtype != torch.bfloat16 or norm_weight.dtype != torch.bfloat16:
        raise ValueError("x and norm_weight must be bfloat16")
    H = x.shape[-1]
    if norm_weight.numel() != H or H % 8 != 0:
        raise ValueError("norm_weight must have one entry per column and the width must be a multiple of 8")
    x2 = _as2d(x).contiguous()
    M = x2.shape[0]
    y = torch.empty_like(x2)
    invar = torch.empty((M,), dtype=torch.float32, device=x.device)
    _lib.call("pf8_rms_norm_fwd", _p(x2), _p(norm_weight.contiguous()), C.c_float(float(epsilon)), M, H, _p(y), _p(invar), _stream())
    return y.reshape(x.shape), invar.reshape(x.shape[:-1])


def fused_rms_norm_ext_grad(x: torch.Tensor, norm_weight: torch.Tensor, invvar: torch.Tensor, dy: torch.Tensor, epsilon: float):
    """paddle._C_ops.fused_rms_norm_ext_grad(x, norm_w, invvar, dy, eps) -> (dx bf16, dw fp32 [H])
    (transformers/fp8_utils.py:528, 739)."""
    for t, n in ((x, "x"), (norm_weight, "norm_weight"), (invvar, "invvar"), (dy, "dy")):
        _dev(t, n)
    if x.dtype != torch.bfloat16 or dy.dtype != torch.bfloat16 or norm_weight.dtype != torch.bfloat16:
        raise ValueError("x, dy and norm_weight must be bfloat16")
    H = x.shape[-1]
    x2, d2 = _as2d(x).contiguous(), _as2d(dy).contiguous()
    if x2.shape != d2.shape:
        raise ValueError("x and dy must have the same shape")
    M = x2.shape[0]
    iv = invvar.reshape(-1).float().contiguous()
    if iv.numel() != M:
        raise ValueError("invvar must have one entry per row")
    dx = torch.empty_like(x2)
    dw = torch.zeros((H,), dtype=torch.float32, device=x.device)
    ws_rows = min(1024, max(int(M), 1))
    ws = torch.empty((ws_rows, H), dtype=torch.float32, device=x.device)      # per-workgroup shares of dw
    _lib.call("pf8_rms_norm_bwd", _p(x2), _p(norm_weight.contiguous()), _p(iv), _p(d2), M, H, _p(dx), _p(dw), _p(ws), ws_rows, _stream())
    return dx.reshape(x.shape), dw


# ---------------------------------------------------------------------------------------------
# moe_permute / moe_unpermute (paddle.nn.functional in the reference)
# ---------------------------------------------------------------------------------------------


_PERMUTE_FLAGS = {}      # device index -> int32[1], OR of the flags of every moe_permute since the last check


def _permute_flag(dev: torch.device) -> torch.Tensor:
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    t = _PERMUTE_FLAGS.get(idx)
    if t is None:
        t = _PERMUTE_FLAGS[idx] = torch.zeros(1, dtype=torch.int32, device=torch.device("cuda", idx))
    return t


def moe_permute_check(device=None) -> None:
    """Read and clear the flag word the `moe_permute` calls on `device` have OR-ed into since the last check
    (one device-to-host copy, i.e. one synchronisation) and raise ValueError when any of them saw routing that
    disagrees with its `tokens_per_expert`."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    t = _permute_flag(dev)
    flags = int(t.item())
    if flags:
        t.zero_()
    if flags & 1:
        raise ValueError("expert_routemap_topk routes more tokens to an expert than tokens_per_expert allows")
    if flags & 2:
        raise ValueError("expert_routemap_topk routes fewer tokens to an expert than tokens_per_expert says")


def moe_permute(hidden_states: torch.Tensor, scale: Optional[torch.Tensor], expert_routemap_topk: torch.Tensor,
                expert_prob_topk: Optional[torch.Tensor], num_experts: int, tokens_per_expert: Sequence[int],
                padding_alignment: int, do_gather: bool = True, validate: bool = False):
    """Gather the routed copies of every token into expert-sorted order, every expert's segment
    padded with zero rows to a multiple of `padding_alignment`.

    cli/train/deepseek_v3_pretrain/moe_utils.py:152-186 (UnZipNode.forward), :217-261 (ZipNode.backward).
    hidden_states bf16 [T, H], or float8_e4m3fn [T, H] with `scale` fp32 [T, H/128];
    expert_routemap_topk int32 [T, topk] (negative = unused slot); expert_prob_topk fp32 [T, topk].
    Returns (hidden_states_unzipped [Mpad, H], zipped_expertwise_rowmap int32 [T, num_experts],
    token_prob_unzipped fp32 [Mpad, 1], scale_unzipped fp32 [Mpad, H/128] or None).
    do_gather=False copies no row: the first result is a `GatheredRows` (the tokens, their scales if they are float8, and
    the source token of every output row), the last is None.
    Counts that do not match the routing (a token routed to an expert beyond its `tokens_per_expert` count is
    dropped; rows of an overstated count are written as zeros) set a sticky flag word that lives on the device for
    the life of the process: the call itself neither allocates nor reads it back, as the reference's operator has no
    device-to-host round trip either.  `moe_permute_check()` reads and clears the flag wherever the caller
    synchronises anyway; `validate=True` does so right after this call (one synchronisation) and raises ValueError.
    """
    _dev(hidden_states, "hidden_states")
    _dev(expert_routemap_topk, "expert_routemap_topk")
    if hidden_states.dim() != 2 or expert_routemap_topk.dim() != 2 or expert_routemap_topk.shape[0] != hidden_states.shape[0]:
        raise ValueError("hidden_states must be [T, H] and expert_routemap_topk [T, topk]")
    is_fp8 = hidden_states.dtype == FP8
    if not is_fp8 and hidden_states.dtype != torch.bfloat16:
        raise ValueError("hidden_states must be bfloat16 or float8_e4m3fn")
    if is_fp8 != (scale is not None):
        raise ValueError("float8 hidden_states come with a scale, bfloat16 hidden_states without")
    T, H = hidden_states.shape
    topk = expert_routemap_topk.shape[1]
    counts = [int(c) for c in tokens_per_expert]
    if len(counts) != num_experts:
        raise ValueError("tokens_per_expert must hold num_experts counts")
    a = int(padding_alignment)
    mpad = sum((c + a - 1) // a * a for c in counts)
    x = hidden_states.contiguous()
    rm = expert_routemap_topk.to(torch.int32).contiguous()
    pr = None if expert_prob_topk is None else expert_prob_topk.to(torch.float32).contiguous()
    dev = x.device
    rowmap = torch.empty((T, num_experts), dtype=torch.int32, device=dev)
    out_p = torch.empty((mpad, 1), dtype=torch.float32, device=dev)
    out_s = None
    xs = None
    if is_fp8:
        if tuple(scale.shape) != (T, H // 128) or scale.dtype != torch.float32:
            raise ValueError("scale must be float32 [T, H/128]")
        xs = scale.contiguous()
    overflow = _permute_flag(dev)
    cnt = (C.c_int64 * num_experts)(*counts)
    if not do_gather:
        src_row = torch.empty((mpad,), dtype=torch.int32, device=dev)
        _lib.call("pf8_moe_permute_map", _p(rm), _p(pr), T, topk, num_experts, cnt, a, _p(rowmap), _p(src_row), _p(out_p), _p(overflow),
                  _stream())
        if validate:
            moe_permute_check(dev)
        return GatheredRows(x, xs, src_row), rowmap, out_p, None
    out_x = torch.empty((mpad, H), dtype=hidden_states.dtype, device=dev)
    if is_fp8:
        out_s = torch.empty((mpad, H // 128), dtype=torch.float32, device=dev)
    _lib.call("pf8_moe_permute", _p(x), int(is_fp8), _p(xs), _p(rm), _p(pr), T, H, topk, num_experts, cnt, a, _p(out_x), _p(rowmap),
              _p(out_p), _p(out_s), _p(overflow), _stream())
    if validate:
        moe_permute_check(dev)
    return out_x, rowmap, out_p, out_s


def moe_unpermute(hidden_states_unzipped: torch.Tensor, zipped_expertwise_rowmap: torch.Tensor, expert_routemap_topk: torch.Tensor,
                  token_prob_unzipped: Optional[torch.Tensor], total_zipped_tokens: int, num_experts: int):
    """Sum the routed copies of every token back (fp32 sum in slot order, bf16 out) and return the
    probabilities in [T, topk] order.  moe_utils.py:188-215 (UnZipNode.backward, ZipNode.forward).
    Returns (hidden_states [T, H] bf16, expert_prob_topk fp32 [T, topk])."""
    _dev(hidden_states_unzipped, "hidden_states_unzipped")
    if hidden_states_unzipped.dtype != torch.bfloat16 or hidden_states_unzipped.dim() != 2:
        raise ValueError("hidden_states_unzipped must be bfloat16 [Mpad, H]")
    T = int(total_zipped_tokens)
    H = hidden_states_unzipped.shape[1]
    topk = expert_routemap_topk.shape[1]
    if tuple(zipped_expertwise_rowmap.shape) != (T, num_experts) or expert_routemap_topk.shape[0] != T:
        raise ValueError("zipped_expertwise_rowmap must be [T, num_experts] and expert_routemap_topk [T, topk]")
    u = hidden_states_unzipped.contiguous()
    rowmap = zipped_expertwise_rowmap.to(torch.int32).contiguous()
    rm = expert_routemap_topk.to(torch.int32).contiguous()
    pu = None if token_prob_unzipped is None else token_prob_unzipped.to(torch.float32).contiguous()
    out = torch.empty((T, H), dtype=torch.bfloat16, device=u.device)
    out_p = torch.empty((T, topk), dtype=torch.float32, device=u.device)
    _lib.call("pf8_moe_unpermute", _p(u), _p(rowmap), _p(rm), _p(pu), T, H, topk, num_experts, _p(out), _p(out_p), _stream())
    return out, out_p
