"""SiluAndMul (python/sglang/srt/layers/activation.py:55-65): x [.., 2d] -> [.., d]."""
import torch

from ..custom_op import CustomOp
from ..ops_backend import get_ops


class SiluAndMul(CustomOp):
    def forward_hip(self, x: torch.Tensor) -> torch.Tensor:
        if not x.is_contiguous():
            x = x.contiguous()
        return get_ops().silu_and_mul(x)


class GeluTanhAndMul(CustomOp):
    """gelu_tanh(gate) * up with gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))); gate and up are
    column blocks of one projection's output."""

    def forward_hip(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        return get_ops().gelu_tanh_and_mul(gate, up)
