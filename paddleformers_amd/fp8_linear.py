"""Host mirror of cli/train/deepseek_v3_pretrain/fp8_linear.py:54-141: the inference-style linear on
pre-quantised block-FP8 weights (`weight._scale` = `weight_scale_inv` [ceil(in/128), ceil(out/128)]).

The reference replaces paddle.nn.functional.linear by fp8_linear for the whole process; here the function
is only exported, and `Linear` calls it.  Only the single-device `Linear` is mirrored: the column/row
(sequence-)parallel subclasses differ from it by their base classes' collectives alone."""
from __future__ import annotations

from typing import Literal, Optional

import torch

from . import kernel as K8

__all__ = ["Linear", "fp8_linear", "register_scale"]

gemm_impl: Literal["bf16", "fp8"] = "bf16"
block_size = 128


def original_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """paddle.nn.functional.linear: y = x . W + b with W stored [in_features, out_features]."""
    y = torch.matmul(x, weight)
    return y if bias is None else y + bias


def fp8_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, name=None) -> torch.Tensor:
    """fp8_linear.py:54-89.  A weight wider than one byte goes to the plain linear; an e4m3 weight is
    either dequantized (gemm_impl == "bf16", the default) and multiplied in bf16, or the activation is
    1x128-quantized and multiplied by the block-scaled FP8 GEMM."""
    if weight.element_size() > 1:
        return original_linear(x, weight, bias)
    if gemm_impl == "bf16":
        return original_linear(x, K8.weight_dequant(weight, weight._scale), bias)
    xq, scale = K8.act_quant(x, block_size)
    # the reference transposes the weight on every call (fp8_linear.py:81 -> kernel.py:194-197); the
    # transposed copy is kept on the weight and redone when the weight or its scales were replaced or
    # written to
    key = (weight.data_ptr(), weight._version, weight._scale.data_ptr(), weight._scale._version)
    cached = getattr(weight, "_pf8_nk", None)
    if cached is None or cached[0] != key:
        bt = weight.view(torch.uint8).t().contiguous().view(K8.FP8)
        cached = (key, bt, weight._scale.t().contiguous())
        weight._pf8_nk = cached
    y = K8._gemm_nk(xq, scale, cached[1], cached[2])
    if bias is not None:
        y += bias
    return y


def register_scale(self):
    """fp8_linear.py:95-106: a one-byte weight gets its fp32 `weight_scale_inv`, one scale per
    block_size x block_size block, also reachable as `weight._scale`."""
    if self.weight.element_size() == 1:
        in_features, out_features = self.weight.shape
        scale_out_features = (out_features + self.block_size - 1) // self.block_size
        scale_in_features = (in_features + self.block_size - 1) // self.block_size
        self.weight_scale_inv = torch.nn.Parameter(
            torch.ones((scale_in_features, scale_out_features), dtype=torch.float32, device=self.weight.device), requires_grad=False)
        self.weight._scale = self.weight_scale_inv


class Linear(torch.nn.Module):
    """fp8_linear.py:109-113 over transformers/linear_utils.Linear (= paddle.nn.Linear): weight
    [in_features, out_features] of `dtype` (an e4m3 dtype makes it a pre-quantised layer, filled by the
    checkpoint loader together with weight_scale_inv), optional bias in bf16."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, dtype=torch.bfloat16, device="cuda", **kwargs):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        one_byte = torch.empty((), dtype=dtype).element_size() == 1
        w = torch.zeros((in_features, out_features), dtype=torch.uint8 if one_byte else dtype, device=device)
        if one_byte:
            w = w.view(dtype)
        else:
            torch.nn.init.normal_(w, std=0.02)
        self.weight = torch.nn.Parameter(w, requires_grad=not one_byte)
        self.bias = torch.nn.Parameter(torch.zeros((out_features,), dtype=torch.bfloat16 if one_byte else dtype, device=device)) if bias else None
        self.block_size = kwargs.get("block_size", 128)
        register_scale(self)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return fp8_linear(x, self.weight, self.bias)
