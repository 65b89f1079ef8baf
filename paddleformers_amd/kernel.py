"""Host mirror of cli/train/deepseek_v3_pretrain/kernel.py: the three operators the inference-style FP8
linear path calls (act_quant, weight_dequant, fp8_gemm), same names, arguments and assertions, on the
library's HIP kernels.  The reference's Triton kernels compute in the default dtype (bfloat16 in its
recipes); so do these."""
from __future__ import annotations

from typing import Tuple

import torch

from . import deep_gemm
from . import functional as F8

FP8 = torch.float8_e4m3fn

__all__ = ["act_quant", "weight_dequant", "fp8_gemm"]


def act_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """kernel.py:51-70 (kernel :29-48): per 1x128 tile s = max|x| / 448, y = x / s cast to e4m3.
    x: contiguous bf16 [..., K], K divisible by block_size -> (y e4m3 [..., K], s fp32 [..., K/128])."""
    assert x.is_contiguous(), "Input tensor must be contiguous"
    assert x.shape[-1] % block_size == 0, f"Last dimension size must be divisible by block_size (block_size={block_size})"
    if block_size != 128:
        raise ValueError("only block_size=128 is supported")
    y, s = F8.fp8_quant_blockwise(x, quant_method="1x128", input_transpose=False, output_scale_transpose=False)
    return y.reshape(x.shape), s.reshape(*x.shape[:-1], x.shape[-1] // block_size)


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """kernel.py:100-118 (kernel :73-97): y[i, j] = x[i, j] * s[i // 128, j // 128], any M and N."""
    return F8.weight_dequant(x, s, block_size)


def fp8_gemm(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor) -> torch.Tensor:
    """kernel.py:190-220 (kernel :129-187): c[..., N] = sum over 128-blocks of K of
    (a_blk . b_blk) * a_s[..., kb] * b_s[kb, n // 128], fp32 accumulation, bf16 result.
    a e4m3 [..., K] with a_s fp32 [..., K/128]; b e4m3 [K, N] (the weight as stored) with b_s [K/128, N/128].
    Like the reference, the weight and its scales are transposed to [N, K] / [N/128, K/128] first."""
    bt = b.view(torch.uint8).t().contiguous().view(FP8)
    bst = b_s.t().contiguous()
    assert a.is_contiguous() and bt.is_contiguous(), "Input tensors must be contiguous"
    assert a_s.is_contiguous() and bst.is_contiguous(), "Scaling factor tensors must be contiguous"
    return _gemm_nk(a, a_s, bt, bst)


def _gemm_nk(a, a_s, bt, bst):
    """The GEMM on a weight already laid out [N, K] with scales [ceil(N/128), K/128]."""
    K = a.shape[-1]
    M = a.numel() // K if K else 0
    N = bt.shape[0]
    c = torch.empty((*a.shape[:-1], N), dtype=torch.bfloat16, device=a.device)
    if M and N:
        deep_gemm.fp8_gemm_nt((a.reshape(M, K), a_s.reshape(M, K // 128)), (bt, bst), c.view(M, N))
    return c
