"""The two forward-context fields the MoE path reads (``_EXTRA_CTX.moe_comm_method`` and
``.moe_comm_type``; reference: ``vllm_ascend/ascend_forward_context.py:280-341``).  On one
GPU the communication method is always all-gather, whose prepare/finalize are the identity."""
from __future__ import annotations

from enum import Enum
from types import SimpleNamespace


class MoECommType(Enum):
    ALLGATHER = 0
    MC2 = 1
    ALLTOALL = 2
    FUSED_MC2 = 3


_EXTRA_CTX = SimpleNamespace(moe_comm_method=None, moe_comm_type=MoECommType.ALLGATHER)


def select_moe_comm_method(*_args, **_kwargs) -> MoECommType:
    """One device, no expert parallelism: all-gather (``ascend_forward_context.py:313-314``)."""
    return MoECommType.ALLGATHER
