"""The single-device orchestration of the fused FP8 MoE layer: unzip -> expert MLP -> zip, forward and backward.

Mirror of `FusionMlpNode` in cli/train/deepseek_v3_pretrain/moe_layer.py:705-1125, the caller that strings
`UnZipNode`, `FP8GroupGemmMlpFunctionNode` and `ZipNode` together between the dispatch and the combine of the expert-
parallel all-to-all.  The all-to-all halves of the reference's layer (`Fp8DispatchQuantNode`, `Fp8CombineQuantNode`,
moe_layer.py:526-700, and `FusionMoeNode` around them) exchange tokens between GPUs and are not part of this build.

Same constructor arguments, attributes and method names; `custom_map` is any object with
  .experts                                    list of objects with bf16 tensors w1 [H, 2I], w2 [I, H]
  .token_dispatcher._comm_manager.tokens_per_expert   routed rows per local expert (unpadded), read at every forward
  .config.seq_length, .config.num_experts_per_tok, .config.adaptive_remained_O1_recompute_ratio
Tensors are torch tensors on the GPU; nothing here records autograd history (the reference drives forward and backward
by hand from its pipeline schedule).

Sub-batched forward / backward (`mlp_fwd_subbatch_rows`, `mlp_bwd_subbatch_rows`): the reference runs the expert MLP
on slices of the unzipped rows and adds every slice's rows into an fp32 token buffer with paddlefleet's
`tokens_zip_unique_add_with_subbatch`, casting to bf16 at the end.  Here the slices write into one bf16 [rows, H] buffer
and the rows are summed per token once, by the same `moe_unpermute` the one-shot path uses: what sub-batching is for (the
up+gate output and the activations of one slice at a time) is kept, the result equals the one-shot path's to the bit,
and the summation order is the documented one (a token's copies in slot order, fp32) instead of slice order.
"""
from __future__ import annotations

from typing import Optional, Tuple, Union

import torch

from . import functional as F8
from .fp8_utils import FP8GroupGemmMlpFunctionNode, extract_first_if_tuple
from .moe_utils import UnZipNode, ZipNode

_Tokens = Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]


def _split_list_prefix(counts, start, end):
    """Rows of every expert's segment that fall into [start, end) (moe_layer.py:838-852)."""
    out, pos = [], 0
    for c in counts:
        lo, hi = max(start, pos), min(end, pos + c)
        out.append(max(0, hi - lo))
        pos += c
    return out


class FusionMlpNode:
    """unzip -> FP8 expert MLP (optionally in sub-batches) -> zip; backward in the reverse order (moe_layer.py:705-1125)."""

    def __init__(self, custom_map, max_topk, recompute_fwd_gate_up=False, is_split_group_gemm=True, dsv3_use_fp8_dispatch=True,
                 mlp_fwd_subbatch_rows=0, mlp_bwd_subbatch_rows=0, output_subbatch_rows=0):
        self.token_dispatcher = custom_map.token_dispatcher
        self.experts = custom_map.experts
        self.unzip_node = UnZipNode()
        self.zip_node = ZipNode()
        self.experts_group_gemm_node = FP8GroupGemmMlpFunctionNode(
            custom_map, recompute_fwd_gate_up=recompute_fwd_gate_up, is_split_group_gemm=is_split_group_gemm)
        self.dsv3_use_fp8_dispatch = dsv3_use_fp8_dispatch
        self.seq_length = custom_map.config.seq_length
        self.num_experts_per_tok = custom_map.config.num_experts_per_tok
        self.adaptive_remained_O1_recompute_ratio = custom_map.config.adaptive_remained_O1_recompute_ratio
        self.recompute_fwd_gate_up = recompute_fwd_gate_up
        self.dispatched_indices = None
        self.dispatched_probs = None
        self.tokens_per_expert = None
        self.padding_token_per_experts = None
        self.router_topk = max_topk
        self.mlp_fwd_subbatch_rows = mlp_fwd_subbatch_rows
        self.mlp_bwd_subbatch_rows = mlp_bwd_subbatch_rows
        self.output_subbatch_rows = output_subbatch_rows     # granularity of the reference's fp32 zip; unused here (see module text)
        self.unzipped_probs = None
        self._src_row = None
        self.m_indices = None
        # with one grouped launch per GEMM (is_split_group_gemm=False) the reordering copies no row.  Forward: the up+gate
        # GEMM and the transposed quantizer of the weight gradient read the dispatched tokens (bf16 tokens quantized per
        # token first) through the row map.  Backward: the gradient tokens are quantized per token, the dgrad GEMM reads them through the map and the
        # transposed quantizer reads the bf16 tokens through it.  Same results to the bit; the expert-sorted copies of the
        # tokens, of the gradients and of their scales never exist.  False = copy.
        self.fuse_unzip = True

    def set_recompute_fwd_gate_up(self, recompute_fwd_gate_up):
        self.experts_group_gemm_node.recompute_fwd_gate_up = recompute_fwd_gate_up

    def reset_statue(self):            # the reference's spelling; its schedule calls this name
        self.dispatched_indices = None
        self.dispatched_probs = None
        self.tokens_per_expert = None
        self.padding_token_per_experts = None
        self.router_topk = None
        self.unzip_node = None
        self.zip_node = None
        self.unzipped_probs = None
        self.m_indices = None
        self.experts_group_gemm_node.reset_statue()
        self.experts_group_gemm_node = None

    # ---- sub-batches ---------------------------------------------------------------------------------------------
    def prepare_env_subbatch(self, unzipped_tokens=None, unzipped_tokens_scale=None, is_fwd=True):
        node = self.experts_group_gemm_node
        if is_fwd:
            assert unzipped_tokens is not None and (unzipped_tokens_scale is not None or isinstance(unzipped_tokens, F8.GatheredRows))
            node.input_fp8 = unzipped_tokens
            node.input_scale = unzipped_tokens_scale
            self.m_indices = node.gen_m_indices(self.padding_token_per_experts)
            node.fwd_subbatch = True
        else:
            if self.m_indices is None:
                self.m_indices = node.gen_m_indices(self.padding_token_per_experts)
            node.bwd_subbatch = True

    def _subbatch_rows(self, total_unzipped_tokens, num_experts, limit):
        rows = min((total_unzipped_tokens // num_experts) // 128 * 128, limit)
        return max(128, rows // 128 * 128)

    def gemm_forward_subbatch(self, unzipped_tokens, unzipped_tokens_scale, unzipped_probs, output, padding_token_per_experts,
                              start_idx, end_idx):
        """The expert MLP on rows [start_idx, end_idx) of the unzipped tokens, written into the same rows of `output`
        (moe_layer.py:791-826; the zip happens once, after the last slice)."""
        start_idx, end_idx = max(0, start_idx), min(unzipped_tokens.shape[0], end_idx)
        sl = slice(start_idx, end_idx)
        node = self.experts_group_gemm_node
        # the grouped launch takes its experts from the m_indices slice, and the node derives its own full-length m_indices
        # (what a one-shot backward uses) from the counts it is handed: the full list, as the reference passes; the
        # expert-by-expert loop (is_split_group_gemm) needs the slice's own counts
        counts = _split_list_prefix(padding_token_per_experts, start_idx, end_idx) if node.is_split_group_gemm else padding_token_per_experts
        rows = unzipped_tokens[sl] if isinstance(unzipped_tokens, F8.GatheredRows) else (unzipped_tokens[sl], unzipped_tokens_scale[sl])
        output[sl] = node.forward(rows, unzipped_probs[sl], counts, m_indices=self.m_indices[sl])
        return output

    def gemm_backward_subbatch(self, unzipped_grad, output, padding_token_per_experts, start_idx, end_idx, reset_status=False):
        """The expert MLP's backward on rows [start_idx, end_idx) (moe_layer.py:828-885); returns the slice's
        probability gradients."""
        node = self.experts_group_gemm_node
        rows = extract_first_if_tuple(unzipped_grad).shape[0]
        start_idx, end_idx = max(0, start_idx), min(rows, end_idx)
        sl = slice(start_idx, end_idx)
        grad = (unzipped_grad[0][sl].contiguous(), unzipped_grad[1][sl].contiguous()) if isinstance(unzipped_grad, tuple) \
            else unzipped_grad[sl].contiguous()
        dx, probs_grad = node.backward(
            grad, self.unzipped_probs[sl].contiguous(), _split_list_prefix(padding_token_per_experts, start_idx, end_idx),
            input_fp8_slice=node.input_fp8[sl].contiguous(),
            input_scale_slice=None if node.input_scale is None else node.input_scale[sl].contiguous(),
            m_indices=self.m_indices[sl].contiguous(), reset_status=reset_status)
        output[sl] = dx
        return probs_grad

    # ---- forward ---------------------------------------------------------------------------------------------------
    @torch.no_grad()
    def forward(self, hs_2d_dispatched: _Tokens, dispatched_indices: torch.Tensor, dispatched_probs: torch.Tensor):
        """hs_2d_dispatched: bf16 tokens [T, H], or (e4m3 tokens, 1x128 scales [T, H/128]) with FP8 dispatch;
        dispatched_indices int [T, topk] (negative = unused slot); dispatched_probs fp32 [T, topk].
        Returns the combined expert outputs, bf16 [T, H]."""
        self.tokens_per_expert = [int(c) for c in self.token_dispatcher._comm_manager.tokens_per_expert]
        self.dispatched_probs = dispatched_probs
        num_experts = len(self.tokens_per_expert)
        padding_token_per_experts = [(x + 127) // 128 * 128 for x in self.tokens_per_expert]
        self.padding_token_per_experts = padding_token_per_experts
        self.dispatched_indices = dispatched_indices.to(torch.int32)
        total_zipped_tokens = extract_first_if_tuple(hs_2d_dispatched).shape[0]
        node = self.experts_group_gemm_node
        map_only = self.fuse_unzip and not node.is_split_group_gemm and not node.use_ue8m0 and total_zipped_tokens > 0
        unzipped_tokens, zipped_expertwise_rowmap, unzipped_probs, unzipped_tokens_scale = self.unzip_node.forward(
            hs_2d_dispatched, self.dispatched_indices, dispatched_probs, topk=self.router_topk, num_experts=num_experts,
            tokens_per_expert=self.tokens_per_expert, do_gather=not map_only)
        self.unzipped_probs = unzipped_probs          # [rows, 1] already
        # the routing is the same in backward: the row map built here also places the gradient tokens
        self._src_row = unzipped_tokens.src_row if map_only else None
        if map_only and not isinstance(hs_2d_dispatched, tuple):
            # bf16 dispatch: the node would quantize every expert-sorted copy of a token (fp8_utils.py:938-941); the 1x128
            # rule is per row, so the T tokens are quantized once instead and read through the map like dispatched FP8 tokens
            unzipped_tokens = unzipped_tokens.quantize(False)
        total_unzipped_tokens = unzipped_tokens.shape[0]
        # adaptive recompute of the up+gate output: on when this rank received more rows than the balanced share times a ratio
        if self.recompute_fwd_gate_up == -1:
            self.set_recompute_fwd_gate_up(
                total_unzipped_tokens > self.seq_length * self.num_experts_per_tok * self.adaptive_remained_O1_recompute_ratio)
        fp8_tokens = isinstance(hs_2d_dispatched, tuple)
        if self.dsv3_use_fp8_dispatch != fp8_tokens:
            raise ValueError("dsv3_use_fp8_dispatch expects (e4m3 tokens, scales) pairs, and only then")
        if fp8_tokens and self.mlp_fwd_subbatch_rows != 0 and total_unzipped_tokens > self.mlp_fwd_subbatch_rows * 2:
            assert node.recompute_fwd_gate_up, "recompute_fwd_gate_up must be true when use_mlp_subbatch = True"
            subbatch_rows = self._subbatch_rows(total_unzipped_tokens, num_experts, self.mlp_fwd_subbatch_rows)
            expert_out = torch.empty((total_unzipped_tokens, unzipped_tokens.shape[1]), dtype=torch.bfloat16, device=unzipped_tokens.device)
            self.prepare_env_subbatch(unzipped_tokens, unzipped_tokens_scale, True)
            for start in range(0, total_unzipped_tokens, subbatch_rows):
                self.gemm_forward_subbatch(unzipped_tokens, unzipped_tokens_scale, unzipped_probs, expert_out,
                                           padding_token_per_experts, start, start + subbatch_rows)
        elif fp8_tokens:
            rows = unzipped_tokens if map_only else (unzipped_tokens, unzipped_tokens_scale)
            expert_out = node.forward(rows, unzipped_probs, padding_token_per_experts)
        else:
            expert_out = node.forward(unzipped_tokens, unzipped_probs, padding_token_per_experts)
        return self.zip_node.forward(expert_out.reshape(-1, expert_out.shape[-1]), zipped_expertwise_rowmap, self.dispatched_indices,
                                     unzipped_probs, total_zipped_tokens=total_zipped_tokens, num_experts=num_experts)

    # ---- backward --------------------------------------------------------------------------------------------------
    @torch.no_grad()
    def backward(self, hidden_states_out_grad: _Tokens):
        """hidden_states_out_grad: bf16 [T, H] or (e4m3, scales).  Returns (gradient of the dispatched tokens bf16 [T, H],
        gradient of the dispatch probabilities fp32 [T, topk]) and drops the node's state."""
        node = self.experts_group_gemm_node
        map_only = self.fuse_unzip and not node.is_split_group_gemm and not node.use_ue8m0 and \
            extract_first_if_tuple(hidden_states_out_grad).shape[0] > 0
        if map_only and getattr(self, "_src_row", None) is not None:
            tok, sc = hidden_states_out_grad if isinstance(hidden_states_out_grad, tuple) else (hidden_states_out_grad, None)
            unzipped_grad = F8.GatheredRows(tok.contiguous(), None if sc is None else sc.contiguous(), self._src_row)
        else:
            unzipped_grad = self.zip_node.backward(hidden_states_out_grad, self.dispatched_indices, self.dispatched_probs,
                                                   top_k=self.router_topk, num_experts=len(self.tokens_per_expert),
                                                   tokens_per_expert=self.tokens_per_expert, do_gather=not map_only)
        total_zipped_tokens = extract_first_if_tuple(hidden_states_out_grad).shape[0]
        total_unzipped_tokens = extract_first_if_tuple(unzipped_grad).shape[0]
        num_experts = len(self.tokens_per_expert)
        padding_token_per_experts = [(x + 127) // 128 * 128 for x in self.tokens_per_expert]
        if self.mlp_bwd_subbatch_rows != 0 and total_unzipped_tokens > self.mlp_bwd_subbatch_rows * 2:
            subbatch_rows = self._subbatch_rows(total_unzipped_tokens, num_experts, self.mlp_bwd_subbatch_rows)
            hidden = extract_first_if_tuple(hidden_states_out_grad).shape[-1]
            dx_rows = torch.empty((total_unzipped_tokens, hidden), dtype=torch.bfloat16, device=self.dispatched_indices.device)
            self.prepare_env_subbatch(is_fwd=False)
            probs_grads = []
            starts = list(range(0, total_unzipped_tokens, subbatch_rows))
            for i, start in enumerate(starts):
                probs_grads.append(self.gemm_backward_subbatch(unzipped_grad, dx_rows, padding_token_per_experts, start, start + subbatch_rows,
                                                               reset_status=i == len(starts) - 1))
            probs_grad = torch.cat([p.reshape(-1) for p in probs_grads])
        else:
            dx_rows, probs_grad = node.backward(unzipped_grad, self.unzipped_probs, padding_token_per_experts)
        hs_dispatched_grad, dispatched_probs_grad = self.unzip_node.backward(dx_rows, total_zipped_tokens, probs_grad, self.dispatched_indices,
                                                                             num_experts=num_experts)
        self.reset_statue()
        return hs_dispatched_grad, dispatched_probs_grad
