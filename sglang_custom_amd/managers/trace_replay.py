"""Replay of a recorded schedule: a caller that dictates, step by step, which requests run and with which tokens,
instead of letting the Scheduler admit and chunk by its own policy.  A step is a list of entries
(request id, next tokens, places among them whose logits are wanted) and the list of requests that end with it.

It is the Scheduler's machinery driven from outside: requests are Req objects, a step is one ScheduleBatch (portions
of prompts as extends over the KV the request already owns -- the chunked-prefill continuation -- and single tokens
either beside them in a mixed batch or, when the step holds nothing else, as a decode batch), one ForwardBatch, one
ModelRunner.forward; KV slots, request rows and state slots come from the runner's pools and go back at a request's
end.  Nothing is sampled: the tokens are given."""
from typing import Dict, List, Optional, Sequence

import torch

from ..model_executor.forward_batch_info import ForwardBatch
from .schedule_batch import Req, ScheduleBatch


class TraceReplayer:
    def __init__(self, model_runner):
        self.mr = model_runner
        self.live: Dict[object, Req] = {}

    def _new_batch(self, reqs: List[Req]) -> ScheduleBatch:
        mr = self.mr
        return ScheduleBatch.init_new(reqs=reqs, req_to_token_pool=mr.req_to_token_pool,
                                      token_to_kv_pool_allocator=mr.token_to_kv_pool_allocator, tree_cache=None,
                                      model_config=mr.model_config)

    @torch.no_grad()
    def step(self, entries: Sequence[dict], end: Sequence[object] = ()) -> Optional[torch.Tensor]:
        """Runs one step; returns the fp32 logits [wanted, vocab] in the order of the entries and of their 'want'
        lists (None when nothing is wanted)."""
        reqs, new_tokens = [], []
        for e in entries:
            toks = [int(t) for t in e["tokens"]]
            if not toks:
                raise ValueError(f"request {e['id']}: an entry without tokens")
            req = self.live.get(e["id"])
            if req is None:
                req = self.live[e["id"]] = Req(e["id"], [])
            reqs.append(req)
            new_tokens.append(toks)
        if len({id(r) for r in reqs}) != len(reqs):
            raise ValueError("a request appears twice in one step")
        logits = None
        if reqs:
            decode = all(len(t) == 1 and r.req_pool_idx is not None for r, t in zip(reqs, new_tokens))
            batch = self._decode_batch(reqs, new_tokens) if decode else self._extend_batch(reqs, new_tokens)
            rows, start = [], 0
            for e, toks in zip(entries, new_tokens):
                for w in e.get("want") or ():
                    if not 0 <= w < len(toks):
                        raise ValueError(f"request {e['id']}: wanted place {w} outside its {len(toks)} tokens")
                    rows.append(start + w)
                start += len(toks)
            fb = ForwardBatch.init_new(batch.get_model_worker_batch(), self.mr)
            if rows:
                fb.logits_rows = torch.tensor(rows, dtype=torch.int64).to(self.mr.device)
            out, _ = self.mr.forward(fb)
            if rows:
                logits = out.requested_logits.float()
        for rid in end:
            self.finish(rid)
        return logits

    def _extend_batch(self, reqs: List[Req], new_tokens: List[List[int]]) -> ScheduleBatch:
        pool = self.mr.req_to_token_pool
        for req, toks in zip(reqs, new_tokens):
            prefix = None
            if req.req_pool_idx is not None:
                # the chunked-prefill continuation: the slots it owns become the prefix of the next extend, under a
                # fresh row of the request table (its state slot stays)
                prefix = pool.req_to_token[req.req_pool_idx, : req.already_computed].clone()
                pool.free(req.req_pool_idx)
                req.req_pool_idx = None
            req.origin_input_ids = req.origin_input_ids + toks
            req.init_next_round_input(prefix)
        batch = self._new_batch(reqs)
        batch.prepare_for_extend()
        return batch

    def _decode_batch(self, reqs: List[Req], new_tokens: List[List[int]]) -> ScheduleBatch:
        batch = ScheduleBatch.for_running(reqs, self.mr.req_to_token_pool, self.mr.token_to_kv_pool_allocator,
                                          self.mr.model_config,
                                          torch.tensor([t[0] for t in new_tokens], dtype=torch.int64).to(self.mr.device))
        batch.prepare_for_decode()
        for req, toks in zip(reqs, new_tokens):
            req.origin_input_ids = req.origin_input_ids + toks
            req.already_computed += 1
        return batch

    def finish(self, rid) -> None:
        """The request gives back its KV slots, its row of the request table and its state slot."""
        req = self.live.pop(rid, None)
        if req is None or req.req_pool_idx is None:
            return
        pool = self.mr.req_to_token_pool
        slots = pool.req_to_token[req.req_pool_idx, : req.already_computed].to(torch.int64)
        self.mr.token_to_kv_pool_allocator.free(slots)
        pool.free(req.req_pool_idx)
        pool.release_state(req)
        req.req_pool_idx = None
