"""ForwardMode / ForwardBatch: the per-forward input record
(python/sglang/srt/model_executor/forward_batch_info.py:61-130, 155-428), field names and
dtypes as the reference passes them:

  input_ids i64 [T]; req_pool_indices i64 [B]; seq_lens i64 [B]; out_cache_loc i64 [T];
  positions i64 [T]; extend_seq_lens / extend_prefix_lens / extend_start_loc i32 [B] (+ _cpu lists)
"""
import dataclasses
from enum import IntEnum, auto
from typing import List, Optional

import torch

from ..ops_backend import get_ops


class ForwardMode(IntEnum):
    EXTEND = auto()         # 1
    DECODE = auto()         # 2
    MIXED = auto()          # 3: chunked prefill + decode requests as extends of length 1
    IDLE = auto()           # 4
    SPLIT_PREFILL = auto()  # 5
    TARGET_VERIFY = auto()  # 6
    DRAFT_EXTEND = auto()   # 7
    DUMMY_FIRST = auto()    # 8

    def is_prefill(self):
        return self.is_extend()

    def is_extend(self):
        return self in (ForwardMode.EXTEND, ForwardMode.MIXED, ForwardMode.DRAFT_EXTEND,
                        ForwardMode.TARGET_VERIFY)

    def is_decode(self):
        return self == ForwardMode.DECODE

    def is_mixed(self):
        return self == ForwardMode.MIXED

    def is_idle(self):
        return self == ForwardMode.IDLE

    def is_decode_or_idle(self):
        return self in (ForwardMode.DECODE, ForwardMode.IDLE)

    def is_cuda_graph(self):
        return self in (ForwardMode.DECODE, ForwardMode.TARGET_VERIFY, ForwardMode.IDLE)


def clamp_position(seq_lens: torch.Tensor) -> torch.Tensor:
    return torch.clamp(seq_lens - 1, min=0).to(torch.int64)


@dataclasses.dataclass
class SequenceStateBatch:
    """One step's view of the per-sequence state (mem_cache.memory_pool.SequenceStatePool) for models whose sequences
    carry state: how the flat token list splits into segments, where each sequence's state lives, and the staging rows
    that the layers fill for the commit at the end of the step (the old state is read by every segment's first token,
    so the new one is written only after the last layer)."""
    pool: object
    req_to_state: torch.Tensor
    req_pool_indices: torch.Tensor
    h_last: torch.Tensor                      # fp32 [layers, B, hidden]
    tok_req: Optional[torch.Tensor] = None    # int32 [T]; None in a decode step (token b is sequence b)
    seg_start: Optional[torch.Tensor] = None  # int32 [B]
    seg_len: Optional[torch.Tensor] = None    # int32 [B]

    def segments(self) -> dict:
        return dict(tok_req=self.tok_req, seg_start=self.seg_start, seg_len=self.seg_len)

    def commit(self, input_ids: torch.Tensor) -> None:
        get_ops().commit_sequence_state(self.pool.rows, self.pool.prev_token, self.h_last, input_ids, self.req_to_state,
                                        self.req_pool_indices, self.seg_start, self.seg_len)


@dataclasses.dataclass
class ForwardBatch:
    forward_mode: ForwardMode
    batch_size: int
    input_ids: torch.Tensor
    req_pool_indices: torch.Tensor
    seq_lens: torch.Tensor
    out_cache_loc: torch.Tensor
    seq_lens_sum: int
    seq_lens_cpu: Optional[torch.Tensor] = None
    return_logprob: bool = False
    positions: torch.Tensor = None
    extend_num_tokens: Optional[int] = None
    extend_seq_lens: Optional[torch.Tensor] = None
    extend_prefix_lens: Optional[torch.Tensor] = None
    extend_start_loc: Optional[torch.Tensor] = None
    extend_prefix_lens_cpu: Optional[List[int]] = None
    extend_seq_lens_cpu: Optional[List[int]] = None
    sampling_info: object = None
    # input-token log-probabilities (forward_batch_info.py:183-190)
    top_logprobs_nums: Optional[List[int]] = None
    extend_logprob_start_lens_cpu: Optional[List[int]] = None
    extend_input_logprob_token_ids_gpu: Optional[torch.Tensor] = None
    req_to_token_pool: object = None
    token_to_kv_pool: object = None
    attn_backend: object = None
    # flat token indices whose logits the caller wants besides every sequence's last one (a replayed trace, scoring);
    # LogitsProcessorOutput.requested_logits answers them
    logits_rows: Optional[torch.Tensor] = None
    seq_state: Optional[SequenceStateBatch] = None
    _token_req_index: Optional[torch.Tensor] = None

    def token_req_index(self) -> Optional[torch.Tensor]:
        """int32 [T]: index in the batch of the sequence each token of an extend belongs to (None in a decode step)."""
        if self.forward_mode.is_decode_or_idle():
            return None
        if self._token_req_index is None:
            dev = self.extend_seq_lens.device
            self._token_req_index = torch.repeat_interleave(
                torch.arange(self.batch_size, dtype=torch.int32, device=dev), self.extend_seq_lens.to(torch.int64),
                output_size=self.extend_num_tokens)
        return self._token_req_index

    def _init_seq_state(self, model_runner) -> None:
        pool = getattr(self.req_to_token_pool, "state_pool", None)
        if pool is None or self.forward_mode.is_idle():
            return
        h_last = torch.empty((pool.layer_num, self.batch_size, pool.hidden), dtype=torch.float32, device=model_runner.device)
        st = SequenceStateBatch(pool=pool, req_to_state=self.req_to_token_pool.req_to_state,
                                req_pool_indices=self.req_pool_indices, h_last=h_last)
        if not self.forward_mode.is_decode():
            st.tok_req = self.token_req_index()
            st.seg_start = self.extend_start_loc
            st.seg_len = self.extend_seq_lens
        self.seq_state = st

    @classmethod
    def init_new(cls, batch, model_runner) -> "ForwardBatch":
        """batch: ModelWorkerBatch (forward_batch_info.py:292-428)."""
        ret = cls(
            forward_mode=batch.forward_mode,
            batch_size=len(batch.seq_lens),
            input_ids=batch.input_ids,
            req_pool_indices=batch.req_pool_indices,
            seq_lens=batch.seq_lens,
            out_cache_loc=batch.out_cache_loc,
            seq_lens_sum=batch.seq_lens_sum,
            seq_lens_cpu=batch.seq_lens_cpu,
            return_logprob=batch.return_logprob,
            sampling_info=batch.sampling_info,
            req_to_token_pool=model_runner.req_to_token_pool,
            token_to_kv_pool=model_runner.token_to_kv_pool,
            attn_backend=model_runner.attn_backend,
        )
        device = model_runner.device
        if ret.forward_mode.is_idle():
            ret.positions = torch.empty((0,), device=device, dtype=torch.int64)
            return ret
        if ret.forward_mode.is_decode():
            ret.positions = batch.positions if batch.positions is not None else clamp_position(batch.seq_lens)
        else:
            ret.extend_seq_lens = torch.tensor(batch.extend_seq_lens, dtype=torch.int32).to(device, non_blocking=True)
            ret.extend_prefix_lens = torch.tensor(batch.extend_prefix_lens, dtype=torch.int32).to(device, non_blocking=True)
            ret.extend_num_tokens = batch.extend_num_tokens
            ret.positions, ret.extend_start_loc = get_ops().compute_position(
                ret.extend_prefix_lens, ret.extend_seq_lens, ret.extend_num_tokens)
            ret.extend_prefix_lens_cpu = batch.extend_prefix_lens
            ret.extend_seq_lens_cpu = batch.extend_seq_lens
            ret.top_logprobs_nums = getattr(batch, "top_logprobs_nums", None)
            ret.extend_logprob_start_lens_cpu = getattr(batch, "extend_logprob_start_lens", None)
            ids = getattr(batch, "extend_input_logprob_token_ids", None)
            if ids is not None:
                ret.extend_input_logprob_token_ids_gpu = ids.to(device, non_blocking=True)
        ret._init_seq_state(model_runner)
        return ret
