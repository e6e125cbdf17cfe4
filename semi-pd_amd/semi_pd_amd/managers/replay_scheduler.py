"""ReplayScheduler: the unified scheduler driven by a trace instead of a sampler.

A trace step names, per request, the next token ids (a portion of its prompt, or one token that an earlier run decoded)
and the places among them whose logits are wanted.  Every step is ONE batch through the same pools, ScheduleBatch
preparation, model runner, decode graphs and kernels that generation uses:

  * a step in which every entry brings one token to a request that already holds tokens is a decode batch
    (ScheduleBatch.prepare_for_decode, the captured decode graphs);
  * anything else is an extend batch in which each request extends its cached prefix -- by a prompt portion or by one
    token, side by side -- exactly how the scheduler continues a chunked prompt: the request's row of req_to_token is
    given back and rebuilt from its slots (prepare_for_extend), new slots come from the allocator.

Nothing is sampled: the logits of the wanted places come back as fp32 rows.  Requests keep their row and slots between
steps (they may sit out a step) and give everything back when the trace ends them, so rows and slots are used again.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from semi_pd_amd.managers.io_struct import SamplingParams
from semi_pd_amd.managers.schedule_batch import Req, ScheduleBatch, host_list_to_device
from semi_pd_amd.managers.scheduler import Scheduler


class ReplayScheduler(Scheduler):
    def __init__(self, server_args, model_runner, tp_rank: int = 0):
        super().__init__(server_args, model_runner, tp_rank, None, None)
        self.live: Dict[str, Req] = {}

    # ------------------------------------------------------------------------------------------ one step
    def replay_step(self, entries: Sequence[dict], end: Sequence[str] = ()) -> Optional[torch.Tensor]:
        """entries: [{"id", "tokens", "want"}]; returns fp32 logits [number of wanted places, vocab] in the order of the
        entries and of their `want` lists (None when nothing is wanted), then releases the requests named in `end`."""
        reqs: List[Req] = []
        news: List[List[int]] = []
        for e in entries:
            tokens = [int(t) for t in e["tokens"]]
            if not tokens:
                continue
            req = self.live.get(e["id"])
            if req is None:
                if len(self.live) >= self.max_running_requests:
                    raise RuntimeError(f"more than {self.max_running_requests} live requests")
                req = Req(e["id"], [], SamplingParams(max_new_tokens=1 << 30, ignore_eos=True))
                self.live[e["id"]] = req
            if len(req.origin_input_ids) + len(tokens) > self.server_args.context_length:
                raise RuntimeError(f"request {e['id']}: longer than the context length {self.server_args.context_length}")
            reqs.append(req)
            news.append(tokens)
        out = None
        if reqs:
            wants = [[int(w) for w in e.get("want", ())] for e in entries if e["tokens"]]
            if all(len(n) == 1 and r.kv_slots for r, n in zip(reqs, news)):
                logits = self._run_decode(reqs, news)
                rows = [i for i, w in enumerate(wants) if w]
                if any(w != [0] for w in wants if w):
                    raise ValueError("a one-token entry can only want place 0")
                out = logits[rows] if rows else None
            else:
                out = self._run_extend(reqs, news, wants)
            self.forward_ct += 1
        for rid in end:
            req = self.live.pop(rid, None)
            if req is not None:
                self.tree_cache.release_req(req)
        return out

    # ------------------------------------------------------------------------------------------ the two batch kinds
    def _run_extend(self, reqs: List[Req], news: List[List[int]], wants: List[List[int]]) -> Optional[torch.Tensor]:
        rows, at = [], 0
        for req, new, want in zip(reqs, news, wants):
            if req.req_pool_idx is not None:
                # like a chunked prompt between its portions: the row goes back, prepare_for_extend rebuilds one from the slots
                self.req_to_token_pool.free(req.req_pool_idx)
                req.req_pool_idx = None
            req.prefix_indices = torch.tensor(req.kv_slots, dtype=torch.int64)
            req.origin_input_ids = req.origin_input_ids + new
            req.fill_ids = list(req.origin_input_ids)
            req.extend_input_len = len(new)
            for w in want:
                if not 0 <= w < len(new):
                    raise ValueError(f"request {req.rid}: wanted place {w} outside its {len(new)} tokens")
                rows.append(at + w)
            at += len(new)
        batch = ScheduleBatch.init_new(reqs, self.req_to_token_pool, self.token_to_kv_pool_allocator, self.tree_cache,
                                       self.device)
        batch.prepare_for_extend()
        # the logits processor gathers these rows of the flat token axis instead of each request's last token
        batch.extend_logit_rows = host_list_to_device(rows or [at - 1], torch.int64, self.device)
        out = self.tp_worker.forward_batch_logits(batch.get_model_worker_batch())
        self.stats["prefill_batches"] += 1
        self.stats["prefill_tokens"] += at
        return out.next_token_logits.float() if rows else None

    def _run_decode(self, reqs: List[Req], news: List[List[int]]) -> torch.Tensor:
        batch = ScheduleBatch.init_new(reqs, self.req_to_token_pool, self.token_to_kv_pool_allocator, self.tree_cache,
                                       self.device)
        lens = [len(r.kv_slots) for r in reqs]
        batch.req_pool_indices = host_list_to_device([r.req_pool_idx for r in reqs], torch.int64, self.device)
        batch.seq_lens = host_list_to_device(lens, torch.int64, self.device)
        batch.seq_lens_cpu, batch.seq_lens_sum = list(lens), sum(lens)
        batch.output_ids = host_list_to_device([n[0] for n in news], torch.int64, self.device)   # the "last sampled" tokens
        batch.prepare_for_decode()
        for req, new in zip(reqs, news):
            req.origin_input_ids = req.origin_input_ids + new
        out = self.tp_worker.forward_batch_logits(batch.get_model_worker_batch())
        self.stats["decode_steps"] += 1
        self.stats["decode_tokens"] += len(reqs)
        return out.next_token_logits.float()
