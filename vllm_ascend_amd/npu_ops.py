"""Stand-ins for the ``torch_npu.npu_*`` operators the fused-MoE path calls, with
the reference's keyword arguments (call sites: ``vllm_ascend/device/device_op.py:103-127,
192-206, 254-291, 950-954``, ``vllm_ascend/quantization/methods/w8a8_dynamic.py:350-351``).
Each one is a thin launcher over libmoe355.so; unsupported options raise."""
from __future__ import annotations

import torch

from . import kernels
from ._lib import W_EKN, W_ENK

ACL_FORMAT_FRACTAL_NZ = 29  # vllm_ascend/utils.py:61


def npu_format_cast(weight: torch.Tensor, acl_format: int = ACL_FORMAT_FRACTAL_NZ) -> torch.Tensor:
    """int8 ``[E, K, N]`` (or ``[K, N]``) -> same logical shape, MFMA-tiled storage.
    The result must only be handed to the grouped-matmul operators."""
    if acl_format != ACL_FORMAT_FRACTAL_NZ:
        raise NotImplementedError(f"npu_format_cast: only FRACTAL_NZ ({ACL_FORMAT_FRACTAL_NZ}) is supported")
    if weight.dim() == 2:
        return kernels.format_cast_nz(weight.unsqueeze(0), W_EKN).squeeze(0)
    return kernels.format_cast_nz(weight, W_EKN)


def format_cast_from_checkpoint(weight_enk: torch.Tensor) -> torch.Tensor:
    """int8 ``[E, N, K]`` (checkpoint order) -> tiled storage, returned with the logical
    shape ``[E, K, N]`` the operators expect.  Same result as transposing and calling
    ``npu_format_cast``, without materialising the transpose."""
    tiled = kernels.format_cast_nz(weight_enk, W_ENK)
    e, n, k = weight_enk.shape
    return tiled.view(e, k, n)


def npu_dynamic_quant(x: torch.Tensor, dst_type: torch.dtype | None = None):
    if dst_type not in (None, torch.int8):
        raise NotImplementedError(f"npu_dynamic_quant: dst_type {dst_type} is not supported (int8 only)")
    return kernels.dynamic_quant(x)


def npu_moe_init_routing_v2(x, expert_idx, *, scale=None, offset=None, active_num=-1, expert_capacity=-1,
                            expert_num=-1, drop_pad_mode=0, expert_tokens_num_type=0, expert_tokens_num_flag=False,
                            quant_mode=-1, active_expert_range=None, row_idx_type=0):
    """-> (expanded_x, expanded_row_idx, expert_tokens, dynamic_scale)."""
    if offset is not None:
        raise NotImplementedError("npu_moe_init_routing_v2: `offset` is not supported")
    if scale is not None and not (quant_mode == -1 and x.dtype == torch.int8):
        raise NotImplementedError("npu_moe_init_routing_v2: `scale` is only supported as the per-token scale of "
                                  "int8 activations that are moved without re-quantisation (quant_mode=-1)")
    if drop_pad_mode != 0 or expert_capacity not in (-1, 0) or row_idx_type != 0:
        raise NotImplementedError("npu_moe_init_routing_v2: drop/pad mode is not supported")
    if quant_mode not in (-1, 1):
        raise NotImplementedError(f"npu_moe_init_routing_v2: quant_mode {quant_mode} is not supported (-1 or 1)")
    if expert_tokens_num_type not in (0, 1):
        raise NotImplementedError("npu_moe_init_routing_v2: expert_tokens_num_type must be 0 (cumsum) or 1 (count)")
    num_rows = expert_idx.numel()
    if active_num not in (-1, 0, num_rows):
        raise NotImplementedError("npu_moe_init_routing_v2: active_num must cover every (token, slot) pair")
    if active_expert_range is not None and list(active_expert_range) != [0, expert_num]:
        raise NotImplementedError("npu_moe_init_routing_v2: a partial active_expert_range (expert parallelism) "
                                  "is not supported on one GPU")
    x2 = x.reshape(-1, x.shape[-1])
    if x.dtype == torch.int8:
        if scale is None or quant_mode != -1:
            raise NotImplementedError("npu_moe_init_routing_v2: int8 activations need their per-token `scale` and "
                                      "quant_mode=-1")
        return kernels.init_routing_prequant(x2, scale.reshape(-1),
                                             expert_idx.reshape(x2.shape[0], expert_idx.shape[-1]), expert_num,
                                             expert_tokens_num_type)
    xs, row_idx, tokens, dyn = kernels.init_routing(x2, expert_idx.reshape(x2.shape[0], expert_idx.shape[-1]), expert_num, quant_mode,
                                                    expert_tokens_num_type)
    return xs, row_idx, tokens, dyn


def npu_grouped_matmul(x, weight, *, bias=None, scale=None, offset=None, antiquant_scale=None, antiquant_offset=None,
                       per_token_scale=None, group_list=None, activation_input=None, activation_quant_scale=None,
                       activation_quant_offset=None, split_item=0, group_type=None, group_list_type=0, act_type=0,
                       output_dtype=None, tuning_config=None):
    """Quantised grouped matmul, the form the down projection uses: one int8 ``x`` [M, K],
    one tiled weight [E, K, N], per-channel ``scale`` [E, N], ``per_token_scale`` [M],
    ``group_type=0`` (split along M), ``split_item`` 2 or 3 (single output).  Returns ``[out]``."""
    if bias is not None or offset is not None or antiquant_scale is not None or antiquant_offset is not None:
        raise NotImplementedError("npu_grouped_matmul: bias / offset / antiquant operands are not supported")
    if group_type != 0 or split_item not in (2, 3) or act_type != 0:
        raise NotImplementedError("npu_grouped_matmul: only group_type=0 with split_item 2/3 is supported")
    xs = x if isinstance(x, (list, tuple)) else [x]
    ws = weight if isinstance(weight, (list, tuple)) else [weight]
    ss = scale if isinstance(scale, (list, tuple)) else [scale]
    ps = per_token_scale if isinstance(per_token_scale, (list, tuple)) else [per_token_scale]
    if len(xs) == 1 and len(ps) == 1 and len(ws) > 1 and len(ws) == len(ss):
        # one tiled [K, N] weight and one [N] scale per expert
        if output_dtype not in (None, torch.bfloat16, torch.float16):
            raise NotImplementedError(f"npu_grouped_matmul: output_dtype {output_dtype} is not supported")
        if isinstance(ws, kernels.ExpertTensorList) and isinstance(ss, kernels.ExpertTensorList):
            weights, scales = ws, ss  # the layer's lists: address tables built at load time
        else:
            weights = list(ws)
            scales = [s_ if s_.dtype == torch.float32 else s_.to(torch.float32) for s_ in ss]
        return [kernels.gmm2_dequant_list(xs[0], weights, scales, ps[0], group_list, group_list_type,
                                          output_dtype or torch.bfloat16)]
    if len(xs) != 1 or len(ws) != 1 or len(ss) != 1 or len(ps) != 1 or ss[0] is None or ps[0] is None:
        raise NotImplementedError("npu_grouped_matmul: expects exactly one x, weight, scale and per_token_scale")
    a, w, s, p = xs[0], ws[0], ss[0], ps[0]
    if a.dtype != torch.int8 or w.dtype != torch.int8:
        raise NotImplementedError("npu_grouped_matmul: only the int8 x int8 form is supported")
    if output_dtype not in (None, torch.bfloat16, torch.float16):
        raise NotImplementedError(
            f"npu_grouped_matmul: output_dtype {output_dtype} is not supported (bfloat16 or float16)")
    k, n = w.shape[1], w.shape[2]
    out = kernels.gmm2_dequant(a, w, s.to(torch.float32), p, group_list, group_list_type, n, k,
                               output_dtype or torch.bfloat16)
    return [out]


def npu_moe_token_unpermute(permuted_tokens, sorted_indices, probs=None, padded_mode=False, restore_shape=None,
                            residual=None):
    """``residual`` (extension): [T, H] tensor added in fp32 before the output is rounded."""
    if padded_mode:
        raise NotImplementedError("npu_moe_token_unpermute: padded_mode is not supported")
    return kernels.token_unpermute(permuted_tokens, sorted_indices, probs, residual)


_ONE_GROUP: dict = {}


def _single_group_list(rows: int, device) -> torch.Tensor:
    key = (rows, str(device))
    t = _ONE_GROUP.get(key)
    if t is None:
        # a fill kernel on the current stream, not a host-to-device copy: no synchronisation, and legal while a
        # HIP graph is being captured (the tensor is created on first use of a row count)
        t = torch.full((1,), rows, dtype=torch.int64, device=device)
        _ONE_GROUP[key] = t
    return t


def npu_quant_matmul(x1, x2, scale, *, offset=None, pertoken_scale=None, bias=None, output_dtype=None):
    """Dense int8 x int8 matmul as the shared expert uses it
    (``vllm_ascend/ops/fused_moe/shared_experts.py:262-301``): ``x1`` int8 ``[M, K]``, ``x2`` int8
    ``[K, N]`` in the tiled storage of :func:`npu_format_cast`, ``scale`` ``[N]``.
    ``output_dtype=torch.int32``: the raw accumulators (scales ignored, as in the reference call);
    ``output_dtype=torch.bfloat16`` / ``torch.float16``: ``half((acc * pertoken_scale[m]) * scale[n])``.
    One expert that owns every row: the grouped kernels with E = 1."""
    if offset is not None or bias is not None:
        raise NotImplementedError("npu_quant_matmul: offset / bias are not supported")
    if x1.dtype != torch.int8 or x2.dtype != torch.int8 or x2.dim() != 2:
        raise NotImplementedError("npu_quant_matmul: int8 [M, K] x int8 [K, N] only")
    lead = x1.shape[:-1]
    a = x1.reshape(-1, x1.shape[-1])
    k, n = x2.shape
    gl = _single_group_list(a.shape[0], a.device)
    w = x2.unsqueeze(0)
    if output_dtype == torch.int32:
        out = kernels.gmm_i32(a, w, gl, 0, n, k, groups_cover_all_rows=True)
    elif output_dtype in (None, torch.bfloat16, torch.float16):
        if pertoken_scale is None:
            raise NotImplementedError("npu_quant_matmul: bf16 / fp16 output needs pertoken_scale")
        out = kernels.gmm2_dequant(a, w, scale.to(torch.float32).reshape(1, n), pertoken_scale.reshape(-1), gl, 0, n, k,
                                   output_dtype or torch.bfloat16)
    else:
        raise NotImplementedError(f"npu_quant_matmul: output_dtype {output_dtype} is not supported")
    return out.reshape(lead + (n,))


def npu_format_cast_int4(packed: torch.Tensor) -> torch.Tensor:
    """int4 weights packed two per byte along N (low nibble = even channel), logical ``[E, K, N]`` held as
    int8 ``[E, K, N/2]`` or its int32 view ``[E, K, N/8]`` (``vllm_ascend/quantization/methods/w4a8.py:313-336``)
    -> same shape and dtype, tiled int4 storage for the W4A8 grouped-matmul operators."""
    if packed.dim() != 3 or packed.dtype not in (torch.int8, torch.uint8, torch.int32):
        raise TypeError("npu_format_cast_int4 expects a packed 3-D int8 / int32 weight")
    per = 8 if packed.dtype == torch.int32 else 2
    e, k, n = packed.shape[0], packed.shape[1], packed.shape[2] * per
    raw = packed.contiguous().view(torch.uint8).reshape(e, k, n // 2)
    tiled = kernels.format_cast_nz_int4(raw, 1, n, k)
    return tiled.view(packed.dtype).reshape(packed.shape)
