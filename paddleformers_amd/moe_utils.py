"""The two reordering nodes either side of the fused FP8 expert MLP, on the permute kernels of libpf8.

Mirror of `UnZipNode` / `ZipNode` in cli/train/deepseek_v3_pretrain/moe_utils.py:130-261 (ERNIE twin:
cli/train/ernie_pretrain/models/moe/token_dispatcher/moe_utils.py): the dispatcher hands each rank its tokens
[T, H] with a top-k routing map; UnZipNode gathers the routed copies into expert-sorted order with every expert's
segment padded to 128 rows (what the contiguous grouped GEMM wants), ZipNode sums the expert outputs back per token.
Their backward passes are each other's forward.  Nothing here records autograd history: the reference drives these
nodes by hand from its schedule, forward and backward as separate calls.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple, Union

import torch

from . import functional as F8

PADDING_ALIGNMENT = 128     # row granularity of the contiguous grouped GEMM (moe_utils.py:160, :235)

_Tokens = Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]


def _permute(tokens: _Tokens, routemap, probs, num_experts, tokens_per_expert, do_gather=True):
    """moe_permute on bf16 tokens or on an (e4m3 tokens, 1x128 scales) pair, as both nodes call it."""
    x, scale = tokens if isinstance(tokens, tuple) else (tokens, None)
    return F8.moe_permute(x, scale, routemap, probs, num_experts=num_experts, tokens_per_expert=tokens_per_expert,
                          padding_alignment=PADDING_ALIGNMENT, do_gather=do_gather)


class UnZipNode:
    """forward: tokens -> expert-sorted padded rows (+ their probabilities, + their scales for FP8 tokens);
    backward: gradient rows -> gradient tokens, summed over each token's routed copies (moe_utils.py:130-199)."""

    def __init__(self, name: str = "unzip"):
        self.name = name
        self.reset_statue()

    def reset_statue(self):            # the reference's spelling; its schedule calls this name
        self.unzipped_probs = None
        self.zipped_expertwise_rowmap = None

    @torch.no_grad()
    def forward(self, hs_2d_dispatched: _Tokens, dispatched_indices: torch.Tensor, dispatched_probs: Optional[torch.Tensor],
                topk: int, num_experts: int, tokens_per_expert: Sequence[int], do_gather: bool = True):
        """do_gather=False (e4m3 tokens only): no row is copied; the first result is the `GatheredRows` the expert MLP
        node reads the tokens through, the last is None."""
        if dispatched_indices.shape[1] != topk:
            raise ValueError(f"dispatched_indices holds {dispatched_indices.shape[1]} slots per token, topk is {topk}")
        rows, rowmap, probs, scale = _permute(hs_2d_dispatched, dispatched_indices, dispatched_probs, num_experts, tokens_per_expert,
                                              do_gather=do_gather)
        self.unzipped_probs, self.zipped_expertwise_rowmap = probs, rowmap
        return rows, rowmap, probs, scale

    @torch.no_grad()
    def backward(self, dx: torch.Tensor, total_zipped_tokens: int, probs_grad: Optional[torch.Tensor],
                 dispatched_indices: torch.Tensor, num_experts: int):
        if self.zipped_expertwise_rowmap is None:
            raise RuntimeError("UnZipNode.backward before forward")
        tokens_grad, probs_grad_topk = F8.moe_unpermute(dx, self.zipped_expertwise_rowmap, dispatched_indices, probs_grad,
                                                        total_zipped_tokens=total_zipped_tokens, num_experts=num_experts)
        self.reset_statue()
        return tokens_grad, probs_grad_topk


class ZipNode:
    """forward: expert output rows -> tokens (fp32 sum of a token's copies in slot order, bf16 out);
    backward: gradient tokens (bf16, or e4m3 with scales) -> expert-sorted padded gradient rows (moe_utils.py:202-261)."""

    def __init__(self, name: str = "zip"):
        self.name = name

    @torch.no_grad()
    def forward(self, expert_out: torch.Tensor, zipped_expertwise_rowmap: torch.Tensor, routemap_topk: torch.Tensor,
                unzipped_probs: Optional[torch.Tensor], total_zipped_tokens: int, num_experts: int) -> torch.Tensor:
        tokens, _ = F8.moe_unpermute(expert_out, zipped_expertwise_rowmap, routemap_topk, unzipped_probs,
                                     total_zipped_tokens=total_zipped_tokens, num_experts=num_experts)
        return tokens

    @torch.no_grad()
    def backward(self, grad_output: _Tokens, dispatched_indices: torch.Tensor, dispatched_probs: Optional[torch.Tensor],
                 top_k: int, num_experts: int, tokens_per_expert: Sequence[int], do_gather: bool = True):
        """do_gather=False: no row is copied; the result is the `GatheredRows` (gradient tokens behind the row map) the
        expert MLP node's backward reads through."""
        rows, _, _, scale = _permute(grad_output, dispatched_indices, dispatched_probs, num_experts, tokens_per_expert, do_gather=do_gather)
        if not do_gather:
            return rows
        return (rows, scale) if isinstance(grad_output, tuple) else rows
