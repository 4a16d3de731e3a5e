"""Device-operator adaptor: the six MoE methods of the reference's
``BaseDeviceAdaptor`` (``vllm_ascend/device/device_op.py:103-127, 133-161, 192-206,
208-234, 254-291, 950-954``) with the same names and keyword arguments, routed to
the MI355X kernels."""
from __future__ import annotations

import torch

from . import npu_ops
from .custom_ops import enable_custom_op


class MI355XDeviceAdaptor:
    @staticmethod
    def npu_moe_init_routing(hidden_states, topk_ids, *, scale=None, active_num: int, expert_num: int,
                             expert_tokens_num_type: int = 1, expert_tokens_num_flag: bool = True,
                             active_expert_range=None, quant_mode: int = -1, act_quant_type=None):
        return npu_ops.npu_moe_init_routing_v2(
            hidden_states, topk_ids, scale=scale, active_num=active_num, expert_num=expert_num,
            expert_tokens_num_type=expert_tokens_num_type, expert_tokens_num_flag=expert_tokens_num_flag,
            active_expert_range=active_expert_range, quant_mode=quant_mode)

    @staticmethod
    def moe_gating_top_k(x, *, k: int, k_group: int, group_count: int, group_select_mode: int, renorm: int,
                         norm_type: int, out_flag: bool, routed_scaling_factor: float = 1.0, eps: float = 1e-20,
                         bias_opt=None, weights_dtype: torch.dtype | None = None):
        """``weights_dtype`` (not in the reference): also have the kernel write the weights in that
        dtype -- the ``topk_weights.to(hidden dtype)`` the caller does next -- and return those."""
        enable_custom_op()
        if weights_dtype is not None and weights_dtype != x.dtype:
            from . import custom_ops, kernels

            custom_ops._check_gating(x, bias_opt)
            _, topk_ids, out, cast = kernels.gating_top_k(x, k, k_group, group_count, group_select_mode, renorm,
                                                          norm_type, out_flag, routed_scaling_factor, eps, bias_opt,
                                                          alt_dtype=weights_dtype)
            return cast, topk_ids, out
        topk_weights, topk_ids, out = torch.ops._C_ascend.moe_gating_top_k(
            x, k=k, k_group=k_group, group_count=group_count, group_select_mode=group_select_mode, renorm=renorm,
            norm_type=norm_type, out_flag=out_flag, routed_scaling_factor=routed_scaling_factor, eps=eps,
            bias_opt=bias_opt)
        return topk_weights, topk_ids.to(torch.int32), out

    @staticmethod
    def npu_dynamic_quant(hidden_states, dynamic_scale=None, *, act_quant_type=torch.int8,
                          use_mxfp_quant: bool = False):
        if use_mxfp_quant:
            raise RuntimeError("MXFP MoE quantization is not available on MI355X in this build.")
        if dynamic_scale is None:
            return npu_ops.npu_dynamic_quant(hidden_states, dst_type=torch.int8)
        return hidden_states, dynamic_scale

    @staticmethod
    def npu_grouped_matmul_swiglu_quant(*, x, weight, group_list, weight_scale, x_scale, bias=None,
                                        use_mxfp_quant: bool = False, act_quant_type=None, weight_quant_type=None,
                                        swiglu_limit: float = 0.0, mxfp_quant_dtype=None, group_list_type: int = 0):
        """``group_list_type`` (not in the reference, whose op only takes a running sum): 1 hands the
        per-expert counts of the dispatcher to the kernel as they are, which saves the cumsum launch."""
        if use_mxfp_quant:
            raise RuntimeError("MXFP MoE quantization is not available on MI355X in this build.")
        enable_custom_op()
        if group_list_type == 1:
            from . import custom_ops, kernels

            custom_ops._reject_unsupported(bias, None)
            if weight_scale.dtype != torch.float32 or weight_scale.dim() != 2:
                # the reference keeps scales in the model dtype and as [E, N, 1]: same conversion as the operator path
                weight_scale = weight_scale.to(torch.float32).reshape(weight.shape[0], -1)
            out, out_scale = kernels.gmm1_swiglu_quant(x, weight, weight_scale, x_scale, group_list, 1,
                                                       weight.shape[2], weight.shape[1], swiglu_limit)
            return out, out_scale, None
        return torch.ops._C_ascend.grouped_matmul_swiglu_quant_weight_nz(
            x=x, weight=weight, weight_scale=weight_scale, x_scale=x_scale, group_list=group_list, bias=bias,
            swiglu_limit=swiglu_limit)

    @staticmethod
    def get_quant_gmm2_kwargs(*, input_dtype, act_quant_type=None, weight_quant_type=None, scale_type=None,
                              per_token_scale_type=None, use_bf16: bool = True, use_mxfp_quant: bool = False) -> dict:
        if use_mxfp_quant:
            raise RuntimeError("MXFP MoE quantization is not available on MI355X in this build.")
        return {"output_dtype": input_dtype if input_dtype in (torch.bfloat16, torch.float16) else torch.bfloat16}

    @classmethod
    def npu_grouped_matmul_gmm2(cls, *, hidden_states, weight, weight_scale, per_token_scale, group_list,
                                group_list_type: int, input_dtype=None, act_quant_type=None, weight_quant_type=None,
                                scale_type=None, per_token_scale_type=None, use_bf16: bool = True,
                                use_mxfp_quant: bool = False, bias=None, fallback_output_dtype=None,
                                mxfp_quant_dtype=None):
        if use_mxfp_quant:
            raise RuntimeError("MXFP MoE quantization is not available on MI355X in this build.")
        if fallback_output_dtype is None:
            first = weight_scale[0] if isinstance(weight_scale, list) else weight_scale
            fallback_output_dtype = first.dtype
        if fallback_output_dtype == torch.float32:
            # fp32 channel scales (the kernels take them in fp32): the product is written in the dtype of the
            # layer's hidden states
            fallback_output_dtype = input_dtype if input_dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
        return npu_ops.npu_grouped_matmul(
            x=[hidden_states], weight=weight, scale=weight_scale, bias=bias, per_token_scale=[per_token_scale],
            split_item=2, group_list_type=group_list_type, group_type=0, group_list=group_list,
            output_dtype=fallback_output_dtype)[0]

    @staticmethod
    def npu_moe_token_unpermute(permuted_tokens, sorted_indices, probs, residual=None):
        # the kernel takes |index| itself (the reference passes torch.abs(sorted_indices))
        return npu_ops.npu_moe_token_unpermute(permuted_tokens=permuted_tokens, sorted_indices=sorted_indices,
                                               probs=probs, residual=residual)


DeviceOperator = MI355XDeviceAdaptor
