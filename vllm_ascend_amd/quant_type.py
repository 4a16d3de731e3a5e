"""Quantisation kinds of the MoE schemes (mirror of ``vllm_ascend/quantization/quant_type.py:26-37``).
Only NONE, W8A8 and W4A8 have kernels on MI355X; the other members exist so that
callers can name them and get a clear NotImplementedError."""
from enum import Enum


class QuantType(Enum):
    NONE = 0
    W8A8 = 1
    W4A8 = 2
    W8A8MXFP = 3
    W4A16 = 4
    W4A4MXFP = 5
    W4A8MXFP = 6
    W8A8FP = 7
    W4A16MXFP = 8


SUPPORTED = (QuantType.W8A8, QuantType.W4A8)
