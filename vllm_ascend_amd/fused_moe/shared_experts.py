"""Shared expert of a W8A8 MoE layer: a dense quantised MLP every token goes through.
Mirrors the int-quantised branch of ``AscendSharedExperts.forward``
(``vllm_ascend/ops/fused_moe/shared_experts.py:254-301``), op for op:
``npu_dynamic_quant`` -> ``npu_quant_matmul`` (int32) -> ``_C_ascend.npu_dequant_swiglu_quant``
(dynamic) -> ``npu_quant_matmul`` (per-token scale, bf16).  On MI355X the dense matmuls are the
grouped kernels with one expert.  With ``multistream_overlap`` the whole MLP runs on a second HIP
stream (default priority) next to the routed experts, fenced by events like the reference's
``before_routed_experts`` / ``wait_stream`` pair."""
from __future__ import annotations

import torch

from .. import npu_ops
from ..custom_ops import enable_custom_op

_SIDE_STREAM = None


def shared_experts_calculation_stream() -> torch.cuda.Stream:
    global _SIDE_STREAM
    if _SIDE_STREAM is None:
        _SIDE_STREAM = torch.cuda.Stream()  # default priority
    return _SIDE_STREAM


class AscendSharedExperts(torch.nn.Module):
    def __init__(self, gate_up_weight: torch.Tensor, gate_up_scale: torch.Tensor, down_weight: torch.Tensor,
                 down_scale: torch.Tensor, swiglu_limit: float = 0.0, multistream_overlap: bool = False,
                 swiglu_alpha: float = 1.0, swiglu_beta: float = 0.0):
        """gate_up_weight int8 [2I, H], down_weight int8 [H, I] (checkpoint order, one row per output
        channel); scales [2I] / [H]."""
        super().__init__()
        enable_custom_op()
        two_i, h = gate_up_weight.shape
        # [N, K] -> logical [K, N] in tiled storage (the reference transposes and casts to NZ)
        self.gate_up_weight = npu_ops.format_cast_from_checkpoint(gate_up_weight.unsqueeze(0)).squeeze(0)
        self.down_weight = npu_ops.format_cast_from_checkpoint(down_weight.unsqueeze(0)).squeeze(0)
        self.gate_up_scale_fp32 = gate_up_scale.reshape(-1).to(torch.float32).contiguous()
        self.down_scale_fp32 = down_scale.reshape(-1).to(torch.float32).contiguous()
        self.swiglu_limit = swiglu_limit
        self.swiglu_alpha = swiglu_alpha
        self.swiglu_beta = swiglu_beta
        self.multistream_overlap = multistream_overlap

    def _mlp(self, hidden_states: torch.Tensor, quantized=None) -> torch.Tensor:
        original_dtype = hidden_states.dtype
        # quantized: (int8 rows, scales) of these hidden states when the caller has them already (the routed
        # experts quantise the same rows with the same per-token rule)
        quantized_x, pertoken_scale = quantized if quantized is not None else npu_ops.npu_dynamic_quant(hidden_states)
        acc = npu_ops.npu_quant_matmul(quantized_x, self.gate_up_weight, self.gate_up_scale_fp32,
                                       pertoken_scale=None, bias=None, output_dtype=torch.int32)
        quantized_x, swiglu_out_scale = torch.ops._C_ascend.npu_dequant_swiglu_quant(
            x=acc, weight_scale=self.gate_up_scale_fp32, activation_scale=pertoken_scale, bias=None,
            quant_scale=None, quant_offset=None, group_index=None, activate_left=True, quant_mode=1,
            swiglu_mode=1, clamp_limit=self.swiglu_limit, glu_alpha=self.swiglu_alpha, glu_bias=self.swiglu_beta)
        return npu_ops.npu_quant_matmul(quantized_x, self.down_weight, self.down_scale_fp32,
                                        pertoken_scale=swiglu_out_scale, bias=None, output_dtype=original_dtype)

    def forward(self, hidden_states: torch.Tensor, before_routed_experts_evt=None, quantized=None) -> torch.Tensor:
        if not self.multistream_overlap:
            return self._mlp(hidden_states, quantized)
        side = shared_experts_calculation_stream()
        main = torch.cuda.current_stream()
        if before_routed_experts_evt is None:
            before_routed_experts_evt = main.record_event()
        with torch.cuda.stream(side):
            side.wait_event(before_routed_experts_evt)
            out = self._mlp(hidden_states, quantized)
            done = side.record_event()
        hidden_states.record_stream(side)
        if quantized is not None:
            for t in quantized:
                t.record_stream(side)
        out.record_stream(main)
        self._done_evt = done
        return out

    def wait(self) -> None:
        """Make the current stream wait for the side-stream MLP (``wait_stream`` in the reference)."""
        if self.multistream_overlap and getattr(self, "_done_evt", None) is not None:
            torch.cuda.current_stream().wait_event(self._done_evt)
            self._done_evt = None
