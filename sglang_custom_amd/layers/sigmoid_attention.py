"""SigmoidAttention: the per-layer hand-off to the attention backend for causal multi-head attention whose weights are
not normalised over the keys (RadixAttention's role, python/sglang/srt/layers/radix_attention.py:59-108, for a mechanism
the reference does not have):

    weight(i, j) = sigmoid((q_i . k_j) * scale * temp_h + bias_h)   for j <= i,      o_i = sum_j weight(i, j) v_j

temp and bias are one fp32 number per query head.  Query head h reads key / value head h // (heads / kv_heads).  Scores
and weights are fp32 in every dtype."""
import torch
from torch import nn


class SigmoidAttention(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int, scaling: float, layer_id: int, device):
        super().__init__()
        assert num_heads % num_kv_heads == 0
        self.tp_q_head_num, self.tp_k_head_num, self.tp_v_head_num = num_heads, num_kv_heads, num_kv_heads
        self.qk_head_dim, self.v_head_dim = head_dim, v_head_dim
        self.scaling = float(scaling)
        self.layer_id = layer_id
        self.temp = nn.Parameter(torch.ones(num_heads, dtype=torch.float32, device=device), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32, device=device), requires_grad=False)

    def forward(self, q: torch.Tensor, forward_batch, out: torch.Tensor) -> torch.Tensor:
        return forward_batch.attn_backend.forward_sigmoid(q, self, forward_batch, out)
