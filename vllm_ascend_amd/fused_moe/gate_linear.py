"""Router gate in fp32.  Counterpart of ``AscendGateLinear``
(``vllm_ascend/ops/fused_moe/gate_linear.py:24-63``): the gate weight is kept in float32 whatever the model
dtype, the input is widened to float32 and the logits stay float32, because expert selection is sensitive to
the precision of the logits.  ``forward`` returns ``(logits, None)`` like the replicated linear layer it
derives from (the second element is the bias when ``skip_bias_add`` is used, which the gate never does)."""
from __future__ import annotations

import torch

from .. import kernels


class AscendGateLinear(torch.nn.Module):
    def __init__(self, input_size: int, output_size: int, bias: bool = False, out_dtype: torch.dtype | None = None,
                 params_dtype: torch.dtype | None = None, force_fp32_compute: bool = False, prefix: str = "",
                 device="cuda"):
        super().__init__()
        # params_dtype / force_fp32_compute are accepted for signature parity and overridden, as in the reference
        self.input_size = input_size
        self.output_size = output_size
        self.out_dtype = out_dtype
        self.prefix = prefix
        self.weight = torch.nn.Parameter(torch.empty(output_size, input_size, dtype=torch.float32, device=device),
                                         requires_grad=False)
        self.bias = (torch.nn.Parameter(torch.zeros(output_size, dtype=torch.float32, device=device),
                                        requires_grad=False) if bias else None)

    @property
    def weight_fp32(self) -> torch.Tensor:
        return self.weight.data

    def weight_loader(self, param: torch.nn.Parameter, loaded_weight: torch.Tensor) -> None:
        if tuple(loaded_weight.shape) != tuple(param.data.shape):
            raise ValueError(f"{self.prefix or 'gate'}: checkpoint shape {tuple(loaded_weight.shape)} does not fit "
                             f"{tuple(param.data.shape)}")
        param.data.copy_(loaded_weight.to(torch.float32))

    def forward(self, x: torch.Tensor):
        if x.dtype not in (torch.float32, torch.bfloat16, torch.float16):
            x = x.to(torch.float32)  # bf16 and fp16 are widened inside the kernel (exact); anything else here
        logits = kernels.router_gate(x, self.weight.data, None if self.bias is None else self.bias.data)
        return logits, None
