"""Layers around an fp32 residual stream (no counterpart in the reference, whose models keep the residual in the
activation dtype and carry nothing but KV between steps):

  BigramHashEmbedding  token embedding times a scale plus a row of a hashed-bigram table; the previous token of a
                       sequence is state (SequenceStatePool.prev_token)
  ShiftedLayerNorm     weight-only layer norm, optionally followed by the token shift
                       hs_t = h_t + (h_{t-1} - h_t) * mu; the previous token's h is state (one fp32 row per layer)
  GatedResidual        x += sigmoid(g1 + b1) * y1 (+ sigmoid(g2 + b2) * y2) on the fp32 stream

All three are one launch each; the constants (scale, hash multipliers, bucket count, epsilon) are constructor
arguments."""
from typing import Optional

import torch
from torch import nn

from ..ops_backend import get_ops


class BigramHashEmbedding(nn.Module):
    def __init__(self, vocab: int, hidden: int, scale: float, buckets: int, mul_prev: int, mul_cur: int, dtype, device):
        super().__init__()
        self.scale, self.buckets, self.mul_prev, self.mul_cur = float(scale), int(buckets), int(mul_prev), int(mul_cur)
        self.weight = nn.Parameter(torch.zeros(vocab, hidden, dtype=dtype, device=device), requires_grad=False)
        # row `buckets` (the last one) serves a sequence's first token
        self.bigram = nn.Parameter(torch.zeros(buckets + 1, hidden, dtype=dtype, device=device), requires_grad=False)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, forward_batch) -> torch.Tensor:
        st = forward_batch.seq_state
        return get_ops().bigram_embedding(input_ids, self.weight.data, self.bigram.data, st.pool.prev_token, st.req_to_state,
                                          st.req_pool_indices, positions, self.scale, self.mul_prev, self.mul_cur, self.buckets,
                                          **st.segments())


class ShiftedLayerNorm(nn.Module):
    """state_layer: which row set of the state pool holds this layer's previous h (None: plain norm, no shift)."""

    def __init__(self, hidden: int, eps: float, dtype, device, state_layer: Optional[int] = None):
        super().__init__()
        self.eps = float(eps)
        self.state_layer = state_layer
        self.weight = nn.Parameter(torch.ones(hidden, dtype=dtype, device=device), requires_grad=False)
        self.shift = None
        if state_layer is not None:
            self.shift = nn.Parameter(torch.zeros(hidden, dtype=dtype, device=device), requires_grad=False)

    def forward(self, x: torch.Tensor, positions: Optional[torch.Tensor] = None, forward_batch=None):
        """x fp32 [T, hidden] -> h, or (h, hs) for a layer with a shift; both in the weight's dtype."""
        ops = get_ops()
        if self.shift is None:
            return ops.layernorm_shift(x, self.weight.data, self.eps)
        st = forward_batch.seq_state
        return ops.layernorm_shift(x, self.weight.data, self.eps, shift=self.shift.data, state=st.pool.rows[self.state_layer],
                                   req_to_state=st.req_to_state, req_pool_indices=st.req_pool_indices, positions=positions,
                                   h_last=st.h_last[self.state_layer], **st.segments())


class GatedResidual(nn.Module):
    """Holds the two gate biases; the gate logits themselves come out of a projection the caller has merged with
    its other projections of the same input."""

    def __init__(self, hidden: int, dtype, device, branches: int = 2):
        super().__init__()
        self.bias1 = nn.Parameter(torch.zeros(hidden, dtype=dtype, device=device), requires_grad=False)
        self.bias2 = nn.Parameter(torch.zeros(hidden, dtype=dtype, device=device), requires_grad=False) if branches > 1 else None

    def forward(self, x: torch.Tensor, g1: torch.Tensor, y1: torch.Tensor, g2=None, y2=None) -> torch.Tensor:
        get_ops().gated_residual_add(x, g1, self.bias1.data, y1, g2, self.bias2.data if y2 is not None else None, y2)
        return x
