"""Host mirror of cli/train/ernie_pretrain/models/fp8_linear.py:51-589: the ERNIE dense FP8 SwiGLU MLP
(`Fp8FusedMlpFunc`, its memory-saving variant and the `Fp8FusedMlp` layer) with `fp8_gemm` and `padding`,
same names and argument meaning, on the library's HIP kernels.

Unlike the transformers/fp8_utils.py wrappers these return the weight gradients (fp32 from the kernel,
handed to autograd in the weights' dtype) instead of accumulating them into main_grad, and quantize the
weights on every call instead of reading a cache."""
from __future__ import annotations

import numpy
import torch

from . import deep_gemm
from . import functional as F8

__all__ = ["Fp8FusedMlp", "Fp8FusedMlpFunc", "MemEfficientFp8FusedMlpFunc", "fp8_gemm", "padding"]


def fp8_gemm(x_fp8, x_scale, w_fp8, w_scale, is_a_1d_scaled, is_b_1d_scaled, out=None, rtn_dtype=torch.bfloat16):
    """fp8_linear.py:51-100: y[Ka, Nb] = x_fp8[Ka, M] . w_fp8[Nb, M]^T with scales handed over transposed
    ([M/128, rows] for a 1x128-scaled operand); `out` given means accumulate into it.  Both operands
    1x128-scaled: the fp32 weight-gradient GEMM.  A 128x128-scaled second operand: the bf16 forward GEMM.
    Zero-sized operands give zeros."""
    if numpy.prod(x_fp8.shape) == 0 or numpy.prod(w_fp8.shape) == 0:
        y = torch.zeros((x_fp8.shape[0], w_fp8.shape[0]), dtype=rtn_dtype, device=x_fp8.device)
        return out + y if out is not None else y
    if is_a_1d_scaled and is_b_1d_scaled:
        return F8.fp8_gemm_blockwise(a=x_fp8, a_decode_scale=x_scale, b=w_fp8, b_decode_scale=w_scale,
                                     out_dtype=out.dtype if out is not None else rtn_dtype, out=out, accumulate=out is not None,
                                     use_split_accumulator=True, is_a_1d_scaled=True, is_b_1d_scaled=True)
    if out is not None:
        raise ValueError("accumulation is only defined for the 1x128-by-1x128 scaled (weight-gradient) form")
    c = torch.empty((x_fp8.shape[0], w_fp8.shape[0]), dtype=rtn_dtype, device=x_fp8.device)
    deep_gemm.fp8_gemm_nt((x_fp8, x_scale.t()), (w_fp8, w_scale.t()), c)
    return c


def padding(x, axis):
    """fp8_linear.py:103-124: zero-pad `axis` (0 rows, 1 columns) up to the next multiple of 512."""
    n = x.shape[axis]
    if n % 512 != 0:
        padding_size = 512 if (n + 128 - (n % 128)) % 512 != 0 else 128
        pad_size = padding_size - (n % padding_size)
        if axis == 0:
            x = torch.cat([x, torch.zeros([pad_size, x.shape[-1]], dtype=x.dtype, device=x.device)], dim=0)
        else:
            x = torch.cat([x, torch.zeros([x.shape[0], pad_size], dtype=x.dtype, device=x.device)], dim=-1)
    return x


def _quant_rows_and_transposed(t):
    """(q, s^T-layout, q_t, s_t) of a bf16 [M, K] tensor: the row-scaled copy of the tensor itself and the
    column-scaled transposed copy of the tensor zero-padded to a multiple of 512 rows (fp8_linear.py:158-180)."""
    if t.shape[0] % 512 != 0:
        q, s = F8.fp8_quant_blockwise(t, quant_method="1x128", input_transpose=False, output_scale_transpose=True)
        tp = padding(t, 0)
        q_t, s_t = F8.fp8_quant_blockwise(tp, quant_method="1x128", input_transpose=True, output_scale_transpose=True,
                                          return_transpose_only=True)
        return q, s, q_t, s_t
    return F8.fp8_quant_blockwise(t, quant_method="1x128", input_transpose=True, output_scale_transpose=True)


def _transposed_only(t):
    tp = padding(t, 0)
    return F8.fp8_quant_blockwise(tp, quant_method="1x128", input_transpose=True, output_scale_transpose=True, return_transpose_only=True)


def _linear_nt(a_fp8, a_scale_t, w, weight_transposed):
    """a [M, K] (scales [K/128, M]) times the bf16 weight w: w^T quantized [N, K] when weight_transposed
    (w is [K, N]: forward), else w itself as [N, K] (w is [N, K]: dgrad)."""
    if weight_transposed:
        w_fp8, w_scale = F8.fp8_quant_blockwise(w, quant_method="128x128", input_transpose=True, output_scale_transpose=False,
                                                return_transpose_only=True)
    else:
        w_fp8, w_scale = F8.fp8_quant_blockwise(w, quant_method="128x128", input_transpose=False, output_scale_transpose=False)
    out = torch.empty((a_fp8.shape[0], w_fp8.shape[0]), dtype=torch.bfloat16, device=a_fp8.device)
    deep_gemm.fp8_gemm_nt((a_fp8, a_scale_t.T), (w_fp8, w_scale), out)
    return out


def _forward(x2, w1, w2):
    """o1 = x . w1, o2 = swiglu(o1), o3 = o2 . w2 (fp8_linear.py:182-205, 369-396)."""
    x_fp8, x_scale = x2
    o1 = _linear_nt(x_fp8, x_scale, w1, True)
    o2 = F8.swiglu(o1)
    o2_fp8, o2_scale = F8.fp8_quant_blockwise(o2, quant_method="1x128", input_transpose=False, output_scale_transpose=True)
    o3 = _linear_nt(o2_fp8, o2_scale, w2, True)
    return o1, o3


def _backward(do3, x_t_fp8, x_t_scale, w1, o1, w2):
    """fp8_linear.py:237-332 / :438-534: (dx [M, H] bf16, dw1 [H, 2I] fp32, dw2 [I, H] fp32)."""
    o2 = F8.swiglu(o1)
    do3_fp8, do3_scale, do3_t_fp8, do3_t_scale = _quant_rows_and_transposed(do3)
    do2 = _linear_nt(do3_fp8, do3_scale, w2, False)
    o2_t_fp8, o2_t_scale = _transposed_only(o2)
    dw2 = fp8_gemm(o2_t_fp8, o2_t_scale, do3_t_fp8, do3_t_scale, True, True, rtn_dtype=torch.float32)
    do1, _ = F8.swiglu_grad(o1, None, do2)
    do1_fp8, do1_scale, do1_t_fp8, do1_t_scale = _quant_rows_and_transposed(do1)
    dx = _linear_nt(do1_fp8, do1_scale, w1, False)
    dw1 = fp8_gemm(x_t_fp8, x_t_scale, do1_t_fp8, do1_t_scale, True, True, rtn_dtype=torch.float32)
    return dx, dw1, dw2


class Fp8FusedMlpFunc(torch.autograd.Function):
    """fp8_linear.py:127-332: keeps the transposed FP8 input and o1 for the backward pass."""

    @staticmethod
    def forward(ctx, x, w1, w2):
        x_orig_shape = x.shape
        x = x.reshape([-1, x_orig_shape[-1]])
        x_fp8, x_scale, x_t_fp8, x_t_scale = _quant_rows_and_transposed(x)
        o1, o3 = _forward((x_fp8, x_scale), w1, w2)
        if len(x_orig_shape) > 2:
            o3 = o3.reshape([x_orig_shape[0], -1, o3.shape[-1]])
        ctx.saved = (x_t_fp8, x_t_scale, w1, o1, w2, x_orig_shape)
        return o3

    @staticmethod
    def backward(ctx, do3):
        do3 = do3.reshape([-1, do3.shape[-1]]).contiguous()
        x_t_fp8, x_t_scale, w1, o1, w2, x_orig_shape = ctx.saved
        dx, dw1, dw2 = _backward(do3, x_t_fp8, x_t_scale, w1, o1, w2)
        if len(x_orig_shape) > 2:
            dx = dx.reshape([x_orig_shape[0], -1, dx.shape[-1]])
        return dx, dw1.to(w1.dtype), dw2.to(w2.dtype)


class MemEfficientFp8FusedMlpFunc(torch.autograd.Function):
    """fp8_linear.py:335-534: keeps only the row-scaled FP8 input; the backward pass recomputes o1 and
    rebuilds the transposed input from the dequantized FP8 copy."""

    @staticmethod
    def forward(ctx, x, w1, w2):
        x_orig_shape = x.shape
        x = x.reshape([-1, x_orig_shape[-1]])
        x_fp8, x_scale = F8.fp8_quant_blockwise(x, quant_method="1x128", input_transpose=False, output_scale_transpose=True)
        _, o3 = _forward((x_fp8, x_scale), w1, w2)
        if len(x_orig_shape) > 2:
            o3 = o3.reshape([x_orig_shape[0], -1, o3.shape[-1]])
        ctx.saved = (x_fp8, x_scale, w1, w2, x_orig_shape)
        return o3

    @staticmethod
    def backward(ctx, do3):
        do3 = do3.reshape([-1, do3.shape[-1]]).contiguous()
        x_fp8, x_scale, w1, w2, x_orig_shape = ctx.saved
        o1 = _linear_nt(x_fp8, x_scale, w1, True)
        x_dequant = F8.fused_act_dequant(x_fp8, x_scale.T.contiguous())
        x_t_fp8, x_t_scale = _transposed_only(x_dequant)
        dx, dw1, dw2 = _backward(do3, x_t_fp8, x_t_scale, w1, o1, w2)
        if len(x_orig_shape) > 2:
            dx = dx.reshape([x_orig_shape[0], -1, dx.shape[-1]])
        return dx, dw1.to(w1.dtype), dw2.to(w2.dtype)


class Fp8FusedMlp(torch.nn.Module):
    """fp8_linear.py:537-589: bias-free SwiGLU MLP, w1 [hidden, 2 * intermediate] and w2 [intermediate,
    hidden] in bf16; `config` carries hidden_size and intermediate_size."""

    def __init__(self, config, device="cuda"):
        super().__init__()
        self.config = config
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.intermediate_size
        self.w1 = torch.nn.Parameter(torch.empty((self.hidden_size, self.intermediate_size * 2), dtype=torch.bfloat16, device=device))
        self.w2 = torch.nn.Parameter(torch.empty((self.intermediate_size, self.hidden_size), dtype=torch.bfloat16, device=device))
        torch.nn.init.normal_(self.w1, std=0.02)
        torch.nn.init.normal_(self.w2, std=0.02)

    def forward(self, x):
        return Fp8FusedMlpFunc.apply(x, self.w1, self.w2)
