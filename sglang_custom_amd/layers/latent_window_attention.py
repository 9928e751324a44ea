"""LatentWindowAttention: the per-layer hand-off to the attention backend for sliding-window attention over a
latent KV cache with a softmax sink (RadixAttention's role, python/sglang/srt/layers/radix_attention.py:59-108, for a
mechanism the reference does not have).  Holds what the backend reads: head count, latent rank, rope width, how many
of the rope features rotate and at which frequencies, window, scale, layer id, and the per-head sink.

The heads share one cache row per token, [c (rank) | rotated rope key]; queries come in absorbed form (q_nope W_uk
per head, rank wide) with their rope part unrotated, and the result per head is the attention-weighted sum of c,
times sigmoid(gate) when gate logits are given."""
import torch
from torch import nn

from .rotary_embedding import rotate_half_inv_freq


class LatentWindowAttention(nn.Module):
    def __init__(self, num_heads: int, kv_rank: int, rope_dim: int, scaling: float, window: int, layer_id: int,
                 rot_dims: int, rot_base: float, device):
        super().__init__()
        assert 0 <= rot_dims <= rope_dim and rot_dims % 2 == 0 and window > 0
        self.tp_q_head_num = num_heads
        self.kv_rank = kv_rank
        self.rope_dim = rope_dim
        self.rot_dims = rot_dims
        self.scaling = float(scaling)
        self.window = int(window)
        self.layer_id = layer_id
        self.sink = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32, device=device), requires_grad=False)
        self.register_buffer("inv_freq", rotate_half_inv_freq(rot_base, rot_dims).to(device), persistent=False)

    def forward(self, qa: torch.Tensor, qr: torch.Tensor, gate, forward_batch, out: torch.Tensor) -> torch.Tensor:
        return forward_batch.attn_backend.forward_latent_window(qa, qr, gate, self, forward_batch, out)
