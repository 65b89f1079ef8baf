"""Host mirror of the ERNIE token dispatcher's FP8 expert nodes
(cli/train/ernie_pretrain/models/moe/token_dispatcher/fp8_utils.py:56-1437): the masked-layout
ExpertsGroupGemmNode and the contiguous-layout ExpertsGroupGemmContiguousNode.  (ExpertsGroupGemmWLCHNode,
:1439-1517, lays the rows out per expert-parallel rank and is not mirrored.)

Masked layout: every expert owns a fixed capacity of `Mmax` rows of the flat `[E * Mmax, H]` activation
tensor, of which the first `tokens_per_expert[e]` are valid; the grouped GEMMs leave the other rows of
their (zero-initialised) outputs untouched.  Same class, method and argument names as the reference; the
arithmetic runs on the library's HIP kernels (no fallback: without the built library every call raises).

Where the reference chains elementwise operators, the fused kernel with the same arithmetic is used:
  * swiglu -> * probs -> cast bf16 -> 1x128 quant (fp8_utils.py:288-297) is
    fused_weighted_swiglu_act_quant, whose definition is that chain (two bf16 roundings);
  * transpose per expert -> 1x128 quant with transposed scales (fp8_utils.py:573-608, 655-686) is
    fused_transpose_split_quant with equal segments of Mmax rows;
  * the un-fused SwiGLU backward (fp8_utils.py:432-437) is fused_swiglu_weighted_bwd, the kernel the
    `swiglu_probs_bwd` switch selects anyway.
"""
from __future__ import annotations

from typing import List, Sequence

import numpy
import torch

from . import deep_gemm
from . import functional as F8
from .fp8_utils import FP8GroupGemmMlpFunctionNode

__all__ = ["ExpertsGroupGemmNode", "ExpertsGroupGemmContiguousNode", "fused_stack_transpose_quant", "split_group_gemm", "has_config"]


def _get_fp8_weight_and_scale(weight, stacked=False, transpose=False):
    """fp8_utils.py:56-73: the cached quantised weight of the asked orientation."""
    if stacked:
        if transpose:
            return weight.fp8_weight_stacked_transpose, weight.fp8_scale_stacked_transpose
        return weight.fp8_weight_stacked, weight.fp8_scale_stacked
    if transpose:
        return weight.fp8_weight_transpose, weight.fp8_scale_transpose
    return weight.fp8_weight, weight.fp8_scale


def fused_stack_transpose_quant(weight_list, transpose=False):
    """fp8_utils.py:76-91: the cache on the first weight if present, else one stacked 128x128 quantization."""
    if hasattr(weight_list[0], "fp8_weight_stacked"):
        return _get_fp8_weight_and_scale(weight_list[0], stacked=True, transpose=transpose)
    return F8.fused_stack_transpose_quant(weight_list, transpose)


def split_group_gemm(x_fp8, x_scale, w_fp8, w_scale, tokens_per_expert, gemm_out):
    """fp8_utils.py:94-129: one dense FP8 GEMM per expert segment of a contiguous layout."""
    start = 0
    for i, n in enumerate(tokens_per_expert):
        n = int(n)
        if n == 0:
            continue
        end = start + n
        deep_gemm.fp8_gemm_nt((x_fp8[start:end], x_scale[start:end]), (w_fp8[i], w_scale[i]), gemm_out[start:end])
        start = end
    return gemm_out


def has_config(config_map, key):
    """fp8_utils.py:132-133."""
    return bool(config_map is not None and key in config_map and config_map[key])


def _quant_weights(weights: Sequence[torch.Tensor], transpose: bool, stack_quant: bool):
    """[E, N, K] e4m3 + [E, N/128, K/128] scales of the experts' weights, N = columns of a weight when
    `transpose` else its rows.  Without `stack_quant` the reference stacks, transposes and quantizes with
    separate operators (fp8_utils.py:200-209, 276-285, 394-402, 518-526); the result of the 128x128 method
    is the same tensor.  (For the up+gate weights that branch of the reference asks for 1x128 scales,
    which deep_gemm's [E, N/128, K/128] scale shape cannot take; the 128x128 method is used here.)"""
    E = len(weights)
    if stack_quant:
        q, s = fused_stack_transpose_quant(list(weights), transpose=transpose)
    else:
        st = torch.stack(list(weights), dim=0)
        if transpose:
            st = st.transpose(1, 2).contiguous()
        q, s = F8.fp8_quant_blockwise(st.reshape(-1, st.shape[-1]), quant_method="128x128", input_transpose=False,
                                      output_scale_transpose=False)
    return q.reshape(E, -1, q.shape[-1]), s.reshape(E, -1, s.shape[-1])


class ExpertsGroupGemmNode:
    """fp8_utils.py:136-784.  forward / backward of E experts' `down(swiglu(up_gate(x)) * probs)` on the
    masked layout; `custom_map.experts` holds objects with `up_gate_proj.weight` [H, 2I] and
    `down_proj.weight` [I, H] (None entries are skipped), `custom_map.config.fp8_fused_ops_configs` the
    switches `stack_quant` and `swiglu_probs_bwd`.  tokens_per_expert: int32 device tensor [E]."""

    def __init__(self, experts, custom_map, name="moe_experts_node"):
        self.o1 = None
        self.unzipped_tokens = None
        self.custom_map = custom_map
        self.unzipped_probs = None
        self.tokens_per_expert = None
        self.fp8_fused_ops_configs = custom_map.config.fp8_fused_ops_configs
        self.name = name
        # backward (with probs): the SwiGLU backward writes do1 and o2_s in the quantized forms their consumers read (one
        # kernel instead of four, same bytes and scales; probs_grad summed per 128-column tile).  False = the reference's calls.
        self.fuse_bwd_quant = True

    def reset_status(self):
        self.o1 = None
        self.unzipped_tokens = None
        self.unzipped_probs = None
        self.tokens_per_expert = None

    # ---- helpers -------------------------------------------------------------------------------
    def _stack_quant(self) -> bool:
        return has_config(self.fp8_fused_ops_configs, "stack_quant")

    @staticmethod
    def _masked(tokens_per_expert, E: int, device) -> torch.Tensor:
        if not isinstance(tokens_per_expert, torch.Tensor):
            tokens_per_expert = torch.tensor([int(t) for t in tokens_per_expert], dtype=torch.int32, device=device)
        if tokens_per_expert.numel() != E:
            raise ValueError(f"tokens_per_expert must have one entry per expert ({E})")
        return tokens_per_expert.to(device=device, dtype=torch.int32)

    @staticmethod
    def _masked_gemm(a_fp8, a_scale, w_quant, w_scale, masked_m, expected_m, dtype=torch.bfloat16):
        """zeros [E, Mmax, N] then the masked grouped GEMM (rows past masked_m[e] stay zero)."""
        E, Mmax, _ = a_fp8.shape
        out = torch.zeros((E, Mmax, w_quant.shape[1]), dtype=dtype, device=a_fp8.device)
        if numpy.prod(a_fp8.shape) != 0:
            deep_gemm.m_grouped_fp8_gemm_nt_masked((a_fp8, a_scale), (w_quant, w_scale), out, masked_m, int(expected_m))
        return out

    @staticmethod
    def _quant_rows(x2d: torch.Tensor, E: int):
        """1x128 quantization of [E * Mmax, K] bf16 -> e4m3 [E, Mmax, K], scales [E, Mmax, K/128]."""
        q, s = F8.fp8_quant_blockwise(x2d, quant_method="1x128", input_transpose=False, output_scale_transpose=False)
        return q.reshape(E, -1, q.shape[-1]), s.reshape(E, -1, s.shape[-1])

    # ---- forward -------------------------------------------------------------------------------
    def fwd_gate_up(self, x_bf16, expert_w1, expert_w_count, tokens_per_expert):
        """fp8_utils.py:179-234: o1 [E, Mmax, 2I] = x . w1 on the valid rows."""
        w1_t_quant, w1_t_scale = _quant_weights(expert_w1, True, self._stack_quant())
        x2d = x_bf16.reshape(-1, x_bf16.shape[-1])
        if x2d.shape[0] % expert_w_count != 0:
            raise ValueError("the rows of x must split evenly over the experts (masked layout)")
        x_fp8, x_scale = self._quant_rows(x2d, expert_w_count)
        masked_m = self._masked(tokens_per_expert, expert_w_count, x_bf16.device)
        return self._masked_gemm(x_fp8, x_scale, w1_t_quant, w1_t_scale, masked_m, x_fp8.shape[1], x_bf16.dtype)

    def fwd_swiglu(self, o1):
        """fp8_utils.py:236-250."""
        return F8.swiglu(o1)

    def _fwd_down(self, o1, probs, expert_w2, expert_w_count, tokens_per_expert):
        w2_quant, w2_scale = _quant_weights(expert_w2, True, self._stack_quant())
        o1_2d = o1.reshape(-1, o1.shape[-1])
        o2_quant, o2_scale = F8.fused_weighted_swiglu_act_quant(o1_2d, probs)
        o2_quant = o2_quant.reshape(expert_w_count, -1, o2_quant.shape[-1])
        o2_scale = o2_scale.reshape(expert_w_count, -1, o2_scale.shape[-1])
        masked_m = self._masked(tokens_per_expert, expert_w_count, o1.device)
        return self._masked_gemm(o2_quant, o2_scale, w2_quant, w2_scale, masked_m, o2_quant.shape[1], o1.dtype)

    def fwd_down(self, o1, unzipped_probs, expert_w_count, tokens_per_expert):
        """fp8_utils.py:252-311: o3 [E, Mmax, H] = bf16(swiglu(o1) * probs) . w2; returns (o3, probs [E, Mmax, 1])."""
        expert_w2 = [x.down_proj.weight for x in self.custom_map.experts if x is not None]
        unzipped_probs = unzipped_probs.reshape(expert_w_count, -1, 1)
        o3 = self._fwd_down(o1, unzipped_probs.reshape(-1), expert_w2, expert_w_count, tokens_per_expert)
        return o3, unzipped_probs

    def fwd_down_no_probs(self, o1, expert_w2, expert_w_count, tokens_per_expert):
        """fp8_utils.py:313-369: the same without the probability weighting (the reference reads the
        weights from custom_map here as well, whatever expert_w2 holds)."""
        expert_w2 = [x.down_proj.weight for x in self.custom_map.experts if x is not None]
        return self._fwd_down(o1, None, expert_w2, expert_w_count, tokens_per_expert)

    # ---- backward ------------------------------------------------------------------------------
    def _dgrad_down(self, expert_w2, unzipped_grad, tokens_per_expert, expected_m):
        E = len(expert_w2)
        bw_w2_quant, bw_w2_scale = _quant_weights(expert_w2, False, self._stack_quant())
        g_fp8, g_scale = self._quant_rows(unzipped_grad.reshape(-1, unzipped_grad.shape[-1]), E)
        masked_m = self._masked(tokens_per_expert, E, unzipped_grad.device)
        return self._masked_gemm(g_fp8, g_scale, bw_w2_quant, bw_w2_scale, masked_m, expected_m, unzipped_grad.dtype)

    def bwd_down_input(self, expert_w2, unzipped_grad, tokens_per_expert, expected_m, quantized=False):
        """fp8_utils.py:371-439: do2_s = out_grad . w2^T, then the weighted SwiGLU backward.
        Returns (do1 [E, Mmax, 2I], o2_s [E, Mmax, I], probs_grad [E, Mmax]).  quantized: do1 as ((fp8 [E, Mmax, 2I],
        scale [E, Mmax, 2I/128]), (fp8_t list, scale_t list)) and o2_s as (fp8_t list, scale_t list), the forms
        bwd_gate_up_input and the weight gradients take."""
        do2_s = self._dgrad_down(expert_w2, unzipped_grad, tokens_per_expert, expected_m)
        E, Mmax, I = do2_s.shape
        if quantized:
            d_fp8, d_scale, d_t, d_ts, o_t, o_ts, probs_grad = F8.swiglu_weighted_bwd_quant(
                self.o1.reshape(E * Mmax, 2 * I), do2_s.reshape(E * Mmax, I), self.unzipped_probs, [Mmax] * E, False, False,
                output_scale_transpose=False)
            return ((d_fp8.reshape(E, Mmax, 2 * I), d_scale.reshape(E, Mmax, -1)), (d_t, d_ts)), (o_t, o_ts), probs_grad.reshape(E, Mmax)
        do1, probs_grad, o2_s = F8.fused_swiglu_weighted_bwd(self.o1.reshape(E * Mmax, 2 * I), do2_s.reshape(E * Mmax, I),
                                                             self.unzipped_probs)
        return do1.reshape(E, Mmax, 2 * I), o2_s.reshape(E, Mmax, I), probs_grad.reshape(E, Mmax)

    def bwd_down_input_no_prob(self, expert_w2, unzipped_grad, tokens_per_expert, expected_m):
        """fp8_utils.py:441-479: (do2 [E, Mmax, I], o2 = swiglu(o1)).  unzipped_grad may be flat [E * Mmax, H]."""
        o2_s = self.fwd_swiglu(self.o1)
        do2_s = self._dgrad_down(expert_w2, unzipped_grad, tokens_per_expert, expected_m)
        return do2_s, o2_s

    def bwd_swiglu(self, o1, do2):
        """fp8_utils.py:481-496."""
        do1, _ = F8.swiglu_grad(o1, None, do2.reshape(*o1.shape[:-1], -1))
        return do1

    def bwd_gate_up_input(self, do1, expert_w1, tokens_per_expert, expected_m):
        """fp8_utils.py:498-554: dx [E, Mmax, H] = do1 . w1^T."""
        E = len(expert_w1)
        bw_w1_quant, bw_w1_scale = _quant_weights(expert_w1, False, self._stack_quant())
        if isinstance(do1, tuple):              # already quantized row-wise: (fp8 [E, Mmax, 2I], scale [E, Mmax, 2I/128])
            do1_fp8, do1_scale = do1
        else:
            do1_fp8, do1_scale = self._quant_rows(do1.reshape(-1, do1.shape[-1]), E)
        masked_m = self._masked(tokens_per_expert, E, do1_fp8.device)
        return self._masked_gemm(do1_fp8, do1_scale, bw_w1_quant, bw_w1_scale, masked_m, expected_m)

    @staticmethod
    def _wgrad(a, b, expert_w: List[torch.Tensor]):
        """main_grad[e] [Ka, Nb] += a_e^T . b_e over the whole capacity of every expert (rows past the valid
        count are zero in both operands): both operands transposed per expert and 1x128-quantized along
        the rows, then the fp32 weight-gradient GEMM (fp8_utils.py:556-716)."""
        E = len(expert_w)

        def transposed(t):
            if isinstance(t, tuple):            # (fp8_t list, scale_t list): transposed and quantized per expert already
                return t
            t2 = t.reshape(-1, t.shape[-1])
            Mmax = t2.shape[0] // E
            if Mmax % 128 != 0:
                raise ValueError("the capacity per expert must be a multiple of 128 for the weight-gradient GEMM")
            return F8.fused_transpose_split_quant(t2, None, [Mmax] * E, False)

        a_t, sa_t = transposed(a)
        b_t, sb_t = transposed(b)
        FP8GroupGemmMlpFunctionNode._expert_wgrads(a_t, sa_t, b_t, sb_t, expert_w, False)

    def bwd_down_weight(self, out_grad, o2, expert_w2):
        """fp8_utils.py:556-638: dw2[e] [I, H] += o2_e^T . out_grad_e."""
        self._wgrad(o2, out_grad, expert_w2)

    def bwd_gate_up_weight(self, do1, input_x, expert_w1):
        """fp8_utils.py:640-716: dw1[e] [H, 2I] += x_e^T . do1_e."""
        self._wgrad(input_x, do1, expert_w1)

    # ---- entry points --------------------------------------------------------------------------
    @torch.no_grad()
    def forward(self, hs_out, unzipped_probs, tokens_per_expert):
        """fp8_utils.py:718-735.  hs_out bf16 [E * Mmax, H], unzipped_probs [E * Mmax] -> o3 [E, Mmax, H]."""
        expert_w1 = [x.up_gate_proj.weight for x in self.custom_map.experts if x is not None]
        expert_w_count = len(expert_w1)
        o1 = self.fwd_gate_up(hs_out, expert_w1, expert_w_count, tokens_per_expert)
        self.o1 = o1
        o3, unzipped_probs = self.fwd_down(o1=o1, unzipped_probs=unzipped_probs, expert_w_count=expert_w_count,
                                           tokens_per_expert=tokens_per_expert)
        self.unzipped_probs = unzipped_probs
        self.unzipped_tokens = hs_out
        return o3

    @torch.no_grad()
    def backward(self, out_grad, tokens_per_expert, dispatched_indices, expected_m):
        """fp8_utils.py:737-750.  out_grad bf16 [E, Mmax, H] -> (dx [E * Mmax, H], probs_grad [E, Mmax]);
        weight gradients go to each weight's main_grad (or grad)."""
        expert_w2 = [x.down_proj.weight for x in self.custom_map.experts if x is not None]
        expert_w1 = [x.up_gate_proj.weight for x in self.custom_map.experts if x is not None]
        E, Mmax = len(expert_w2), int(numpy.prod(out_grad.shape[:-1])) // max(len(expert_w2), 1)
        fuse = self.fuse_bwd_quant and 0 < E <= 256 and Mmax > 0 and Mmax % 128 == 0 and self.o1.shape[-1] % 256 == 0
        do1, o2_s, probs_grad = self.bwd_down_input(expert_w2, out_grad, tokens_per_expert, expected_m, quantized=fuse)
        do1_rows, do1_t = do1 if fuse else (do1, do1)
        del do1
        dx = self.bwd_gate_up_input(do1_rows, expert_w1, tokens_per_expert, expected_m)
        dx = dx.reshape(-1, dx.shape[-1])
        self.bwd_down_weight(out_grad, o2_s, expert_w2)
        self.bwd_gate_up_weight(do1_t, self.unzipped_tokens, expert_w1)
        self.reset_status()
        return dx, probs_grad

    @torch.no_grad()
    def forward_no_prob(self, hs_out, tokens_per_expert):
        """fp8_utils.py:752-762."""
        expert_w1 = [x.up_gate_proj.weight for x in self.custom_map.experts if x is not None]
        expert_w_count = len(expert_w1)
        expert_w2 = [x.down_proj.weight for x in self.custom_map.experts if x is not None]
        o1 = self.fwd_gate_up(hs_out, expert_w1, expert_w_count, tokens_per_expert)
        self.o1 = o1
        o3 = self.fwd_down_no_probs(o1, expert_w2, expert_w_count, tokens_per_expert)
        self.unzipped_tokens = hs_out
        return o3

    @torch.no_grad()
    def backward_no_prob(self, out_grad, tokens_per_expert):
        """fp8_utils.py:764-784.  The capacity is the row count of out_grad divided by the experts."""
        expert_w2 = [x.down_proj.weight for x in self.custom_map.experts if x is not None]
        expert_w1 = [x.up_gate_proj.weight for x in self.custom_map.experts if x is not None]
        expected_m = int(numpy.prod(out_grad.shape[:-1]) // len(expert_w1))
        out_grad = out_grad.reshape(-1, out_grad.shape[-1])
        do2, o2_s = self.bwd_down_input_no_prob(expert_w2, out_grad, tokens_per_expert, expected_m)
        do1 = self.bwd_swiglu(self.o1, do2)
        dx = self.bwd_gate_up_input(do1, expert_w1, tokens_per_expert, expected_m)
        dx = dx.reshape(-1, dx.shape[-1])
        self.bwd_down_weight(out_grad, o2_s, expert_w2)
        self.bwd_gate_up_weight(do1, self.unzipped_tokens, expert_w1)
        self.reset_status()
        return dx


class ExpertsGroupGemmContiguousNode:
    """fp8_utils.py:787-1437.  The same expert MLP on the contiguous layout: rows sorted by expert, every
    expert's segment a multiple of 128 rows (tokens_per_expert, a list of ints).  Switches read from
    custom_map.config.fp8_fused_ops_configs: stack_quant, split_group_gemm, spaq (fused SwiGLU + quantize
    with power-of-two scales), swiglu_probs_bwd, transpose_split_quant (fused, power-of-two scales).
    dequant_input keeps the quantised input instead of the bf16 one and rebuilds it for the weight
    gradient; a2a_async_fn(dx) -> (dx, task), when given to backward, is started right after dx is ready
    and waited for at the end."""

    def __init__(self, custom_map, recompute_fwd_gate_up=False, dequant_input=False, group=None,
                 name="experts_group_gemm_contiguous_node"):
        self.custom_map = custom_map
        self.recompute_fwd_gate_up = recompute_fwd_gate_up
        self.dequant_input = dequant_input
        self.tokens_per_expert = None
        self.m_indices = None
        self.unzipped_probs = None
        self.input = None
        self.input_fp8 = None
        self.input_scale = None
        self.o1 = None
        self.fp8_fused_ops_configs = custom_map.config.fp8_fused_ops_configs
        self.is_split_group_gemm = has_config(self.fp8_fused_ops_configs, "split_group_gemm")
        self.group = group
        self.name = name
        # backward quantizes out_grad twice (row-wise for the dgrad GEMM, transposed per expert for the weight gradient)
        # and do1 and o2_s right after the SwiGLU backward has written them; with this set the first pair comes from
        # one read of out_grad and the SwiGLU backward writes only the quantized forms (same bytes and scales as the
        # reference's sequence; probs_grad summed per 128-column tile).  False = the reference's sequence of calls.
        self.fuse_bwd_quant = True

    def reset_status(self):
        self.tokens_per_expert = None
        self.m_indices = None
        self.unzipped_probs = None
        self.input = None
        self.input_fp8 = None
        self.input_scale = None
        self.o1 = None

    def gen_m_indices(self, tokens_per_expert):
        """fp8_utils.py:854-873: expert id of every row, int32."""
        counts = torch.tensor([int(t) for t in tokens_per_expert], dtype=torch.int64)
        return torch.repeat_interleave(torch.arange(len(counts), dtype=torch.int32), counts).cuda()

    def _stack_quant(self) -> bool:
        return has_config(self.fp8_fused_ops_configs, "stack_quant")

    def _grouped(self, a_fp8, a_scale, w_quant, w_scale, out):
        if numpy.prod(a_fp8.shape) != 0:
            if self.is_split_group_gemm:
                split_group_gemm(a_fp8, a_scale, w_quant, w_scale, self.tokens_per_expert, out)
            else:
                deep_gemm.m_grouped_fp8_gemm_nt_contiguous((a_fp8, a_scale), (w_quant, w_scale), out, self.m_indices)
        return out

    def fwd_gate_up(self, x, expert_w1, num_expert, tokens_per_expert, scale=None):
        """fp8_utils.py:875-947.  x: bf16 [M, H]; e4m3 with its `scale` (needs dequant_input); or None to
        reuse the cached quantised input."""
        self.tokens_per_expert = tokens_per_expert
        if not self.is_split_group_gemm:
            self.m_indices = self.gen_m_indices(tokens_per_expert)
        w1_t_quant, w1_t_scale = _quant_weights(expert_w1, True, self._stack_quant())
        if x is None:
            x_fp8, x_scale = self.input_fp8, self.input_scale
            assert x_fp8 is not None and x_scale is not None
        elif scale is not None:
            x_fp8, x_scale = x, scale
            assert self.dequant_input, "If a scale is provided, it indicates that a2a is using fp8. Dequant_input must be enabled."
        else:
            x_fp8, x_scale = F8.fp8_quant_blockwise(x, quant_method="1x128", input_transpose=False, output_scale_transpose=True)
            x_scale = x_scale.T
        o1 = torch.empty((x_fp8.shape[0], w1_t_quant.shape[1]), dtype=expert_w1[0].dtype, device=x_fp8.device)
        self._grouped(x_fp8, x_scale, w1_t_quant, w1_t_scale, o1)
        if self.dequant_input:
            self.input_fp8 = x_fp8
            self.input_scale = x_scale
        else:
            self.input = x
        return o1

    def fwd_swiglu(self, o1):
        return F8.swiglu(o1)

    def fwd_down(self, o1, unzipped_probs, expert_w2, num_expert):
        """fp8_utils.py:953-1017: (o3 [M, H], probs [M, 1]).  `spaq` quantizes with power-of-two scales."""
        w2_quant, w2_scale = _quant_weights(expert_w2, True, self._stack_quant())
        o2_fp8, o2_scale = F8.fused_weighted_swiglu_act_quant(o1, unzipped_probs,
                                                              using_pow2_scaling=has_config(self.fp8_fused_ops_configs, "spaq"))
        unzipped_probs = unzipped_probs.unsqueeze(-1)
        o3 = torch.empty((o2_fp8.shape[0], w2_quant.shape[1]), dtype=o1.dtype, device=o1.device)
        self._grouped(o2_fp8, o2_scale, w2_quant, w2_scale, o3)
        return o3, unzipped_probs

    def bwd_down_input(self, expert_w2, unzipped_grad, o1, quantized=False):
        """fp8_utils.py:1019-1094: (do1 [M, 2I], o2_s [M, I], probs_grad [M]).  unzipped_grad: bf16, or its row-wise
        (fp8, scale [H/128, M]) pair.  quantized: do1 comes back as ((fp8, scale [2I/128, M]), (fp8_t list, scale_t list))
        and o2_s as (fp8_t list, scale_t list), the forms bwd_gate_up_input and the weight gradients take."""
        bw_w2_quant, bw_w2_scale = _quant_weights(expert_w2, False, self._stack_quant())
        if isinstance(unzipped_grad, tuple):
            g_fp8, g_scale = unzipped_grad
        else:
            g_fp8, g_scale = F8.fp8_quant_blockwise(unzipped_grad, quant_method="1x128", input_transpose=False, output_scale_transpose=True)
        do2_s = torch.empty((g_fp8.shape[0], bw_w2_quant.shape[1]), dtype=o1.dtype, device=o1.device)
        self._grouped(g_fp8, g_scale.T, bw_w2_quant, bw_w2_scale, do2_s)
        if quantized:
            pow2 = has_config(self.fp8_fused_ops_configs, "transpose_split_quant")
            d_fp8, d_scale, d_t, d_ts, o_t, o_ts, probs_grad = F8.swiglu_weighted_bwd_quant(
                o1, do2_s, self.unzipped_probs.squeeze(-1), self.tokens_per_expert, False, pow2)
            return ((d_fp8, d_scale), (d_t, d_ts)), (o_t, o_ts), probs_grad
        do1, probs_grad, o2_s = F8.fused_swiglu_weighted_bwd(o1, do2_s, self.unzipped_probs.squeeze(-1))
        return do1, o2_s, probs_grad

    def bwd_swiglu(self, o1, do2):
        do1, _ = F8.swiglu_grad(o1, None, do2)
        return do1

    def bwd_gate_up_input(self, do1, expert_w1):
        """fp8_utils.py:1100-1155: dx [M, H]."""
        bw_w1_quant, bw_w1_scale = _quant_weights(expert_w1, False, self._stack_quant())
        if isinstance(do1, tuple):              # already quantized row-wise: (fp8, scale [2I/128, M])
            do1_fp8, do1_scale = do1
        else:
            do1_fp8, do1_scale = F8.fp8_quant_blockwise(do1, quant_method="1x128", input_transpose=False, output_scale_transpose=True)
        dx = torch.empty((do1_fp8.shape[0], bw_w1_quant.shape[1]), dtype=torch.bfloat16, device=do1_fp8.device)
        self._grouped(do1_fp8, do1_scale.T, bw_w1_quant, bw_w1_scale, dx)
        return dx

    def fused_transpose_split_quant(self, x, tokens_per_expert, pow_2_scales):
        """fp8_utils.py:1157-1180."""
        return F8.fused_transpose_split_quant(x, None, tokens_per_expert, pow_2_scales)

    def _wgrad(self, a, b, expert_w):
        """fp8_utils.py:1182-1319: per expert, a_e^T . b_e into main_grad (or grad).  Without the
        `transpose_split_quant` switch the reference transposes the whole tensor, quantizes it 1x128 with
        plain scales and splits the scales per expert: the same values as the per-expert kernel without
        power-of-two scales, since every segment is a multiple of 128 rows."""
        pow2 = has_config(self.fp8_fused_ops_configs, "transpose_split_quant")
        # an operand handed in as (fp8_t list, scale_t list) was transposed and quantized (with this switch's scales) already
        a_t, sa_t = a if isinstance(a, tuple) else self.fused_transpose_split_quant(a, self.tokens_per_expert, pow2)
        b_t, sb_t = b if isinstance(b, tuple) else self.fused_transpose_split_quant(b, self.tokens_per_expert, pow2)
        FP8GroupGemmMlpFunctionNode._expert_wgrads(a_t, sa_t, b_t, sb_t, expert_w, pow2)

    def bwd_down_weight(self, do3, o2, expert_w2):
        self._wgrad(o2, do3, expert_w2)

    def bwd_gate_up_weight(self, do1, input_x, expert_w1):
        self._wgrad(input_x, do1, expert_w1)

    @torch.no_grad()
    def forward(self, hs_out, unzipped_probs, tokens_per_expert, origin_token_per_experts, scale=None):
        """fp8_utils.py:1321-1343."""
        self.origin_token_per_experts = origin_token_per_experts
        if hs_out.shape[0] == 0:
            self.unzipped_probs = unzipped_probs.unsqueeze(-1)
            return torch.zeros_like(hs_out)
        expert_w1 = [x.up_gate_proj.weight for x in self.custom_map.experts if x is not None]
        expert_w2 = [x.down_proj.weight for x in self.custom_map.experts if x is not None]
        num_expert = len(expert_w1)
        o1 = self.fwd_gate_up(hs_out, expert_w1, num_expert, tokens_per_expert, scale=scale)
        if not self.recompute_fwd_gate_up:
            self.o1 = o1
        o3, unzipped_probs = self.fwd_down(o1, unzipped_probs, expert_w2, num_expert)
        self.unzipped_probs = unzipped_probs
        return o3

    @torch.no_grad()
    def backward(self, out_grad, a2a_async_fn=None):
        """fp8_utils.py:1345-1436: (dx, probs_grad); zero rows still create the gradient accumulators."""
        if out_grad.shape[0] == 0:
            dx = torch.zeros_like(out_grad)
            probs_grad = torch.zeros_like(self.unzipped_probs)
            for expert in self.custom_map.experts:
                if expert is None:
                    continue
                for w in (expert.down_proj.weight, expert.up_gate_proj.weight):
                    if hasattr(w, "main_grad"):
                        if w.main_grad is None:
                            w.main_grad = torch.zeros(w.shape, dtype=torch.float32, device=w.device)
                    elif w.grad is None:
                        w.grad = torch.zeros(w.shape, dtype=torch.float32, device=w.device)
            if a2a_async_fn:
                dx, task = a2a_async_fn(dx)
                task.wait()
            return dx, probs_grad
        expert_w2 = [x.down_proj.weight for x in self.custom_map.experts if x is not None]
        expert_w1 = [x.up_gate_proj.weight for x in self.custom_map.experts if x is not None]
        if self.recompute_fwd_gate_up:
            o1 = self.fwd_gate_up(None if self.dequant_input else self.input, expert_w1, len(expert_w1), self.tokens_per_expert)
        else:
            o1 = self.o1
        rows = [int(t) for t in self.tokens_per_expert]
        fuse = (self.fuse_bwd_quant and not self.is_split_group_gemm and len(rows) <= 256 and all(r % 128 == 0 for r in rows)
                and o1.shape[1] % 256 == 0 and out_grad.dtype == torch.bfloat16 and out_grad.shape[1] % 128 == 0)
        do1_rows = do1_t = None
        if fuse:
            pow2 = has_config(self.fp8_fused_ops_configs, "transpose_split_quant")
            g_fp8, g_scale, g_t, g_ts = F8.quant_and_transpose_split(out_grad, rows, False, pow2)
            (do1_rows, do1_t), o2_s, probs_grad = self.bwd_down_input(expert_w2, (g_fp8, g_scale), o1, quantized=True)
            out_grad = (g_t, g_ts)
        else:
            do1, o2_s, probs_grad = self.bwd_down_input(expert_w2, out_grad, o1)
            do1_rows = do1_t = do1
            del do1
        del o1
        if not self.recompute_fwd_gate_up:
            self.o1 = None
        if self.dequant_input:
            input_x = F8.fused_act_dequant(self.input_fp8, self.input_scale)
            self.input_scale = None
        else:
            input_x = self.input
        task = None
        if a2a_async_fn is None:
            self.bwd_gate_up_weight(do1_t, input_x, expert_w1)
            del input_x
            if not self.dequant_input:
                self.input = None
            dx = self.bwd_gate_up_input(do1_rows, expert_w1)
            del do1_rows, do1_t
            self.bwd_down_weight(out_grad, o2_s, expert_w2)
        else:
            dx = self.bwd_gate_up_input(do1_rows, expert_w1)
            dx, task = a2a_async_fn(dx)
            self.bwd_gate_up_weight(do1_t, input_x, expert_w1)
            del input_x
            if not self.dequant_input:
                self.input = None
            del do1_rows, do1_t
            self.bwd_down_weight(out_grad, o2_s, expert_w2)
            task.wait()
        self.reset_status()
        return dx, probs_grad
