"""Continuous-batching scheduler.

Semantics follow the reference scheduler (vllm/v1/core/sched/scheduler.py:69):

- No prefill/decode phases: each request's ``num_computed_tokens`` catches
  up to ``num_tokens`` under a shared token budget (chunked prefill falls
  out of the clamp).
- RUNNING requests are scheduled first; on allocation failure the
  lowest-priority (last) running request is preempted by evicting all its
  blocks and requeuing it.
- WAITING requests join while budget, seats, and KV blocks remain;
  prefix-cache lookups skip already-cached prompt prefixes.
- FCFS or priority policy.
"""

from __future__ import annotations

import heapq
from collections import deque
from typing import Optional

from vllm_amd.config import EngineConfig
from vllm_amd.core.kv_cache_manager import KVCacheManager
from vllm_amd.core.sched_output import (
    CachedRequestData,
    EngineCoreOutput,
    ModelRunnerOutput,
    NewRequestData,
    SchedulerOutput,
    SchedulerStats,
)
from vllm_amd.request import Request, RequestStatus



class PriorityWaiting:
    """Heap-backed waiting queue with the deque surface schedule() uses
    ([0], popleft, append, appendleft, remove, len, iter). Ordering is
    Request.__lt__ = (priority, arrival). appendleft (preemption
    requeue) is just a push: the heap restores priority order, which is
    exactly what preempted requests need."""

    def __init__(self):
        self._heapq = heapq
        self._h: list = []

    def append(self, request) -> None:
        self._heapq.heappush(self._h, request)

    appendleft = append

    def popleft(self):
        return self._heapq.heappop(self._h)

    def remove(self, request) -> None:
        self._h.remove(request)  # rare (abort); O(n) + heapify
        self._heapq.heapify(self._h)

    def __getitem__(self, idx):
        if idx != 0:
            raise IndexError("PriorityWaiting only exposes the head")
        return self._h[0]

    def __len__(self) -> int:
        return len(self._h)

    def __bool__(self) -> bool:
        return bool(self._h)

    def __iter__(self):
        return iter(sorted(self._h))


class Scheduler:

    def __init__(
        self,
        config: EngineConfig,
        num_gpu_blocks: int,
        num_host_blocks: int = 0,
    ) -> None:
        self.config = config
        sched_cfg = config.scheduler_config
        self.max_num_batched_tokens = sched_cfg.max_num_batched_tokens
        self.max_num_seqs = sched_cfg.max_num_seqs
        self.enable_chunked_prefill = sched_cfg.enable_chunked_prefill
        self.long_prefill_token_threshold = sched_cfg.long_prefill_token_threshold
        self.policy = sched_cfg.policy
        self.max_model_len = config.model_config.max_model_len
        self.block_size = config.cache_config.block_size

        sc = config.scheduler_config
        if sc.num_speculative_tokens > 0:
            if sc.spec_decode_method == "medusa":
                from vllm_amd.spec_decode.medusa import MedusaProposer

                self.spec_proposer = MedusaProposer()
            elif sc.spec_decode_method == "eagle":
                from vllm_amd.spec_decode.eagle import EagleProposer

                self.spec_proposer = EagleProposer()
            elif sc.spec_decode_method == "draft":
                from vllm_amd.spec_decode.draft_model import (
                    DraftModelProposer)

                self.spec_proposer = DraftModelProposer()
            else:
                from vllm_amd.spec_decode.ngram import NgramProposer

                self.spec_proposer = NgramProposer(
                    min_n=sc.ngram_prompt_lookup_min,
                    max_n=sc.ngram_prompt_lookup_max,
                    k=sc.num_speculative_tokens,
                )
        else:
            self.spec_proposer = None
        self.spec_stats_drafted = 0
        self.spec_stats_accepted = 0
        # Dynamic speculation length (role of the reference's dynamic
        # per-batch speculation): start at the configured k, shrink when
        # acceptance is poor (wasted verify compute), grow back toward
        # the configured cap when acceptance is high.
        self.spec_k = sc.num_speculative_tokens
        self._spec_k_max = sc.num_speculative_tokens
        self._spec_window_drafted = 0
        self._spec_window_accepted = 0
        spec = config.model_config.spec
        uniform_window = (spec.sliding_window
                          if spec.sliding_window > 0
                          and spec.global_attn_every_n_layers == 0 else 0)
        enable_caching = config.cache_config.enable_prefix_caching
        if spec.has_row_state or spec.pooling_only:
            # Defense in depth (EngineArgs also clears the flag): SSM
            # state is not content-addressable and encoders need every
            # position's hidden state — a prefix hit would skip tokens
            # those models must actually process.
            enable_caching = False
        self.kv_cache_manager = KVCacheManager(
            num_gpu_blocks=num_gpu_blocks,
            block_size=config.cache_config.block_size,
            enable_caching=enable_caching,
            num_host_blocks=num_host_blocks,
            sliding_window=uniform_window,
            mixed_window=(spec.sliding_window
                          if spec.is_mixed_attn else 0),
        )

        self.requests: dict[str, Request] = {}
        # FCFS: plain deque. Priority: a heap with the same deque-like
        # surface — O(log n) insert instead of re-sorting per add
        # (reference request_queue.py priority queue role).
        self.waiting = (PriorityWaiting() if self.policy == "priority"
                        else deque())
        self.running: list[Request] = []
        # req_ids finished since the last schedule() call; the runner uses
        # this to clear its persistent-batch rows.
        self.finished_req_ids: set[str] = set()
        # Stats
        self.prefix_cache_queries = 0
        self.prefix_cache_hits = 0
        self.num_preemptions_total = 0
        # Multimodal encoder admission budget (encoder tokens whose
        # encode runs start per step; reference encoder-budget role).
        self.max_encoder_tokens = (
            sched_cfg.max_encoder_tokens_per_step
            or sched_cfg.max_num_batched_tokens)
        self.num_encoder_deferrals = 0

    # ------------------------------------------------------------------
    # Request admission / removal

    def add_request(self, request: Request) -> None:
        self.requests[request.request_id] = request
        request.status = RequestStatus.WAITING
        self.waiting.append(request)

    def extend_prompt(self, req_id: str, token_ids: list[int],
                      logit_taps: Optional[list[int]] = None,
                      close: bool = False) -> None:
        """Append prompt tokens to a request admitted with
        prompt_open=True (streamed input). logit_taps are absolute
        positions; close=True ends the stream, after which the request
        samples like any other once its prompt is computed."""
        request = self.requests[req_id]
        request.extend_prompt(token_ids)
        if logit_taps:
            request.logit_taps = sorted(set(request.logit_taps)
                                        | set(logit_taps))
        if close:
            request.prompt_open = False

    def finish_requests(
        self, request_ids: list[str], status: RequestStatus
    ) -> None:
        """Externally finish (abort) requests."""
        for req_id in request_ids:
            request = self.requests.get(req_id)
            if request is None or request.is_finished():
                continue
            if request.status == RequestStatus.RUNNING:
                self.running.remove(request)
            else:
                try:
                    self.waiting.remove(request)
                except ValueError:
                    pass
            request.status = status
            self._free_request(request)

    def has_guided_requests(self) -> bool:
        return any(r.grammar is not None for r in self.running)

    def has_pooling_requests(self) -> bool:
        return any(r.sampling_params.pooling for r in self.running)

    def has_unfinished_requests(self) -> bool:
        return bool(self.waiting or self.running)

    def get_num_unfinished_requests(self) -> int:
        return len(self.waiting) + len(self.running)

    # ------------------------------------------------------------------
    # Scheduling

    def schedule(self) -> SchedulerOutput:  # noqa: C901
        fast = self._try_schedule_decode_fast()
        if fast is not None:
            return fast
        return self._schedule_slow()

    def _try_schedule_decode_fast(self) -> Optional[SchedulerOutput]:
        """Steady-state decode fast path: every running request advances
        exactly one token, nothing is waiting, no spec/grammar state.
        The general loop costs ~20 us of Python per request per step —
        ~20 ms at batch 1024, which out-budgets a ~5 ms TP=8 decode
        step. Here only block-boundary crossings (1 in block_size
        steps) take the full allocate_slots; everything else is O(1)
        bookkeeping. Bails (with rollback) to the general path whenever
        any precondition fails, so semantics are identical by
        construction."""
        running = self.running
        if (self.waiting or not running
                or len(running) > self.max_num_batched_tokens):
            return None
        mgr = self.kv_cache_manager
        if mgr.sliding_window > 0 or mgr.mixed_window > 0:
            return None  # window reclaim stays on the audited path
        bs = self.block_size
        max_len = self.max_model_len
        # Precondition scan (no mutation).
        for r in running:
            if (r.spec_token_ids or r.grammar is not None
                    or r.prompt_open or r.logit_taps
                    or r.num_tokens + r.num_output_placeholders
                    - r.num_computed_tokens != 1
                    or r.num_computed_tokens + 1 > max_len):
                return None
        req_to_blocks = mgr.req_to_blocks
        cached = CachedRequestData()
        req_ids = cached.req_ids
        new_block_ids = cached.new_block_ids
        resumed = cached.resumed
        num_computed_list = cached.num_computed_tokens
        new_token_ids = cached.new_token_ids
        committed: list = []
        ok = True
        for r in running:
            total = r.num_computed_tokens + 1
            blocks_needed = (total + bs - 1) // bs
            if total % bs == 0 or blocks_needed > len(
                    req_to_blocks[r.request_id]):
                nb = mgr.allocate_slots(r, 1)
                if nb is None:
                    ok = False
                    break
                ids = [b.block_id for b in nb]
            else:
                ids = []
            req_ids.append(r.request_id)
            resumed.append(False)
            new_block_ids.append(ids)
            num_computed_list.append(r.num_computed_tokens)
            new_token_ids.append(
                r.all_token_ids[r.num_computed_tokens:total])
            r.num_computed_tokens = total
            if total == r.num_tokens + r.num_output_placeholders:
                r.num_output_placeholders += 1
            committed.append((r, len(ids)))
        if not ok:
            # Roll back and let the general path preempt. Blocks
            # allocated in this failed pass MUST be released too:
            # leaving them in req_to_blocks makes the manager think the
            # request owns them while the runner was never told — its
            # stale block table then silently corrupts block 0.
            for r, n_alloc in committed:
                r.num_computed_tokens -= 1
                # The placeholder was bumped iff (restored computed + 2)
                # == tokens + bumped placeholders.
                if (r.num_computed_tokens + 2
                        == r.num_tokens + r.num_output_placeholders):
                    r.num_output_placeholders -= 1
                mgr.release_trailing(r, n_alloc)
            return None
        n = len(running)
        out = SchedulerOutput(
            scheduled_new_reqs=[],
            scheduled_cached_reqs=cached,
            num_scheduled_tokens={r.request_id: 1 for r in running},
            total_num_scheduled_tokens=n,
            finished_req_ids=self.finished_req_ids,
            scheduled_spec_decode_tokens={},
            kv_swap_ops=mgr.take_swap_ops(),
        )
        self.finished_req_ids = set()
        return out

    def _schedule_slow(self) -> SchedulerOutput:  # noqa: C901
        token_budget = self.max_num_batched_tokens
        scheduled_spec_tokens: dict[str, list[int]] = {}
        scheduled_new_reqs: list[NewRequestData] = []
        cached = CachedRequestData()
        num_scheduled_tokens: dict[str, int] = {}
        preempted_reqs: set[str] = set()
        logit_taps: dict[str, list[int]] = {}

        # ---- RUNNING loop (reference scheduler.py:484) ----
        req_index = 0
        while req_index < len(self.running) and token_budget > 0:
            request = self.running[req_index]
            num_spec = len(request.spec_token_ids)
            num_new_tokens = (request.num_tokens + num_spec
                              + request.num_output_placeholders
                              - request.num_computed_tokens)
            if self.long_prefill_token_threshold > 0:
                num_new_tokens = min(
                    num_new_tokens, self.long_prefill_token_threshold
                )
            num_new_tokens = min(num_new_tokens, token_budget)
            # Don't run past the context window.
            num_new_tokens = min(
                num_new_tokens,
                self.max_model_len - request.num_computed_tokens,
            )
            if num_new_tokens <= 0:
                req_index += 1
                continue

            new_blocks = None
            while True:
                new_blocks = self.kv_cache_manager.allocate_slots(
                    request, num_new_tokens
                )
                if new_blocks is not None:
                    break
                # Preempt the lowest-priority running request (the last one).
                if self.policy == "priority":
                    victim = max(
                        self.running,
                        key=lambda r: (r.priority, r.arrival_time),
                    )
                else:
                    victim = self.running[-1]
                self._preempt(victim)
                preempted_reqs.add(victim.request_id)
                if victim is request:
                    break  # this very request was evicted
            if request.request_id in preempted_reqs:
                # Could not schedule it; it's back in waiting.
                continue

            cached.req_ids.append(request.request_id)
            cached.resumed.append(False)
            cached.new_block_ids.append([b.block_id for b in new_blocks])
            cached.new_block_ids_w.append(
                self.kv_cache_manager.last_w_block_ids(
                    request.request_id, len(new_blocks)))
            cached.num_computed_tokens.append(request.num_computed_tokens)
            taps = request.take_logit_taps(
                request.num_computed_tokens,
                request.num_computed_tokens + num_new_tokens)
            if taps:
                logit_taps[request.request_id] = taps
            # Tokens the runner hasn't seen yet: any output tokens generated
            # since the prompt (runner keeps its own copy; for non-resumed
            # requests only the newest token is unseen).
            cached.new_token_ids.append(
                request.all_token_ids[
                    request.num_computed_tokens : request.num_computed_tokens
                    + num_new_tokens
                ]
            )
            if num_spec > 0:
                scheduled_spec_tokens[request.request_id] = \
                    list(request.spec_token_ids)
                request.spec_token_ids = []
            num_scheduled_tokens[request.request_id] = num_new_tokens
            token_budget -= num_new_tokens
            # Advance optimistically at schedule time (async scheduling:
            # the next schedule() may run before this step's results).
            request.num_computed_tokens += num_new_tokens
            if (request.num_computed_tokens
                    == request.num_tokens + request.num_output_placeholders
                    and not request.prompt_open):
                request.num_output_placeholders += 1
            req_index += 1

        # ---- WAITING loop (reference scheduler.py:692) ----
        encoder_budget = self.max_encoder_tokens
        while (
            self.waiting
            and token_budget > 0
            and len(self.running) < self.max_num_seqs
            and not preempted_reqs  # don't admit while evicting
        ):
            request = self.waiting[0]
            resumed = request.status == RequestStatus.PREEMPTED
            if (request.encoder_tokens > 0
                    and request.num_computed_tokens == 0
                    and request.encoder_tokens > encoder_budget
                    and encoder_budget < self.max_encoder_tokens):
                # Budget partially spent and this request would start
                # another encode run: defer to the next step (FCFS order
                # holds). A request bigger than the WHOLE budget still
                # admits alone — otherwise it could never run.
                self.num_encoder_deferrals += 1
                break

            # Prefix-cache lookup for fresh requests.
            new_computed_blocks = []
            num_computed = request.num_computed_tokens
            # mean-pooling and prompt_logprobs need hidden states /
            # logits of EVERY prompt position — cached prefixes cannot
            # be skipped.
            skip_cache = (request.sampling_params.pooling == "mean"
                          or bool(request.sampling_params.prompt_logprobs))
            if num_computed == 0 and not resumed and not skip_cache:
                (
                    new_computed_blocks,
                    num_computed,
                ) = self.kv_cache_manager.get_computed_blocks(request)
                self.prefix_cache_queries += request.num_tokens
                self.prefix_cache_hits += num_computed
            elif resumed:
                # Preemption dropped all blocks; try the prefix cache to
                # recover whatever is still resident.
                (
                    new_computed_blocks,
                    num_computed,
                ) = self.kv_cache_manager.get_computed_blocks(request)

            num_new_tokens = request.num_tokens - num_computed
            if self.long_prefill_token_threshold > 0:
                num_new_tokens = min(
                    num_new_tokens, self.long_prefill_token_threshold
                )
            if num_new_tokens > token_budget:
                if not self.enable_chunked_prefill:
                    break
                num_new_tokens = token_budget
            if num_new_tokens <= 0:
                break

            new_blocks = self.kv_cache_manager.allocate_slots(
                request, num_new_tokens, new_computed_blocks
            )
            if new_blocks is None:
                break  # out of KV blocks; stop admitting

            self.waiting.popleft()
            self.running.append(request)
            request.status = RequestStatus.RUNNING
            if request.encoder_tokens > 0 and num_computed == 0:
                encoder_budget -= request.encoder_tokens
            request.num_computed_tokens = num_computed

            all_block_ids = self.kv_cache_manager.get_block_ids(
                request.request_id
            )
            all_block_ids_w = self.kv_cache_manager.get_block_ids_w(
                request.request_id
            )
            taps = request.take_logit_taps(
                num_computed, num_computed + num_new_tokens)
            if taps:
                logit_taps[request.request_id] = taps
            if resumed:
                cached.req_ids.append(request.request_id)
                cached.resumed.append(True)
                cached.new_block_ids.append(all_block_ids)
                cached.new_block_ids_w.append(all_block_ids_w)
                cached.num_computed_tokens.append(num_computed)
                cached.new_token_ids.append(list(request.all_token_ids))
            else:
                scheduled_new_reqs.append(
                    NewRequestData(
                        req_id=request.request_id,
                        prompt_token_ids=list(request.all_token_ids),
                        block_ids=all_block_ids,
                        num_computed_tokens=num_computed,
                        sampling_params=request.sampling_params,
                        grammar=request.grammar,
                        lora_id=request.lora_id,
                        mm_data=request.mm_data,
                        block_ids_w=all_block_ids_w,
                        prompt_open=request.prompt_open,
                    )
                )
            num_scheduled_tokens[request.request_id] = num_new_tokens
            token_budget -= num_new_tokens
            request.num_computed_tokens += num_new_tokens
            if (request.num_computed_tokens
                    == request.num_tokens + request.num_output_placeholders
                    and not request.prompt_open):
                request.num_output_placeholders += 1

        if any(self.requests[r].prompt_open for r in cached.req_ids):
            cached.prompt_open = [self.requests[r].prompt_open
                                  for r in cached.req_ids]
        total = sum(num_scheduled_tokens.values())
        out = SchedulerOutput(
            scheduled_new_reqs=scheduled_new_reqs,
            scheduled_cached_reqs=cached,
            num_scheduled_tokens=num_scheduled_tokens,
            total_num_scheduled_tokens=total,
            finished_req_ids=self.finished_req_ids,
            scheduled_spec_decode_tokens=scheduled_spec_tokens,
            kv_swap_ops=self.kv_cache_manager.take_swap_ops(),
            logit_taps=logit_taps,
        )
        self.finished_req_ids = set()
        return out

    def _preempt(self, request: Request) -> None:
        self.running.remove(request)
        self.kv_cache_manager.free(request)
        request.status = RequestStatus.PREEMPTED
        request.num_computed_tokens = 0
        request.num_output_placeholders = 0
        request.spec_token_ids = []
        request.num_preemptions += 1
        self.num_preemptions_total += 1
        self.waiting.appendleft(request)

    # ------------------------------------------------------------------
    # Post-execution update

    def update_from_output(
        self,
        scheduler_output: SchedulerOutput,
        runner_output: ModelRunnerOutput,
    ) -> list[EngineCoreOutput]:
        outputs: list[EngineCoreOutput] = []
        sampled_by_req = dict(
            zip(runner_output.req_ids, runner_output.sampled_token_ids)
        )
        logprobs_by_req = runner_output.logprobs or {}
        pooled_by_req = runner_output.pooled or {}
        plp_by_req = runner_output.prompt_logprobs or {}
        spec_sched = scheduler_output.scheduled_spec_decode_tokens
        requests = self.requests

        for req_id, num_sched in scheduler_output.num_scheduled_tokens.items():
            request = requests.get(req_id)
            if request is None or request.is_finished():
                continue  # aborted mid-step

            pooled_vec = pooled_by_req.get(req_id) if pooled_by_req else None
            if pooled_vec is not None:
                # Pooling request: prefill done, no tokens — finish now.
                request.status = RequestStatus.FINISHED_STOPPED
                outputs.append(EngineCoreOutput(
                    req_id=req_id,
                    new_token_ids=[],
                    finish_reason=request.get_finished_reason(),
                    num_cached_tokens=request.num_cached_tokens,
                    pooled=pooled_vec,
                ))
                self.running.remove(request)
                self._free_request(request)
                continue

            if plp_by_req:
                new_plp = plp_by_req.get(req_id)
                if new_plp and not request.is_finished():
                    request.prompt_logprob_chunks = (
                        getattr(request, "prompt_logprob_chunks", [])
                        + new_plp)

            if runner_output.tapped_logits:
                tapped = runner_output.tapped_logits.get(req_id)
                if tapped is not None:
                    outputs.append(EngineCoreOutput(
                        req_id=req_id, new_token_ids=[],
                        tapped_logits=tapped))

            new_token_ids = sampled_by_req.get(req_id) or []
            num_spec_sched = (len(spec_sched.get(req_id, ()))
                              if spec_sched else 0)
            if num_spec_sched > 0:
                # Roll back KV positions of rejected draft tokens: they
                # were computed from draft values that turned out wrong
                # (reference scheduler.py:1679 spec-token accounting).
                num_rejected = num_spec_sched + 1 - len(new_token_ids)
                if num_rejected > 0:
                    request.num_computed_tokens -= num_rejected
                self.spec_stats_drafted += num_spec_sched
                self.spec_stats_accepted += len(new_token_ids) - 1
                self._spec_window_drafted += num_spec_sched
                self._spec_window_accepted += len(new_token_ids) - 1
                if self._spec_window_drafted >= 64:
                    rate = (self._spec_window_accepted
                            / self._spec_window_drafted)
                    if rate < 0.25 and self.spec_k > 1:
                        self.spec_k -= 1
                    elif rate > 0.7 and self.spec_k < self._spec_k_max:
                        self.spec_k += 1
                    self._spec_window_drafted = 0
                    self._spec_window_accepted = 0
            if not new_token_ids:
                continue  # mid chunked-prefill, nothing sampled

            stopped = False
            kept_tokens: list[int] = []
            for tok in new_token_ids:
                kept_tokens.append(tok)
                request.append_output_token(tok)
                if request.num_output_placeholders:
                    request.num_output_placeholders -= 1
                stopped = self._check_stop(request, tok)
                if stopped:
                    break

            out = EngineCoreOutput(
                req_id=req_id,
                new_token_ids=kept_tokens,
                finish_reason=request.get_finished_reason(),
                stop_reason=request.stop_reason,
                num_cached_tokens=request.num_cached_tokens,
                new_logprobs=logprobs_by_req.get(req_id),
                new_prompt_logprobs=getattr(
                    request, "prompt_logprob_chunks", None),
            )
            request.prompt_logprob_chunks = None
            outputs.append(out)
            if stopped:
                self.running.remove(request)
                self._free_request(request)
            # Spec decode covers sampled requests too: the runner's
            # verify loop is an exact rejection sampler for one-hot
            # drafts (model_runner.py). Grammar requests stay gated —
            # draft positions would need per-position grammar masks.
            elif (self.spec_proposer is not None
                    and request.grammar is None
                    and not request.sampling_params.pooling):
                if getattr(self.spec_proposer, "model_based", False):
                    drafts = (runner_output.draft_token_ids or {}).get(
                        req_id)
                else:
                    drafts = self.spec_proposer.propose(
                        request.all_token_ids)
                # Guard: a draft model with a larger vocab could propose
                # ids the target cannot embed — truncate at the first
                # out-of-range id (later drafts condition on it).
                drafts = (drafts or [])[: self.spec_k]
                vocab = self.config.model_config.spec.vocab_size
                for di, t in enumerate(drafts):
                    if not 0 <= t < vocab:
                        drafts = drafts[:di]
                        break
                request.spec_token_ids = drafts
        return outputs

    def _check_stop(self, request: Request, last_token: int) -> bool:
        params = request.sampling_params
        if (
            request.num_output_tokens >= params.min_tokens
            and not params.ignore_eos
            and request.eos_token_id is not None
            and last_token == request.eos_token_id
        ):
            request.status = RequestStatus.FINISHED_STOPPED
            return True
        if (
            request.num_output_tokens >= params.min_tokens
            and last_token in params.all_stop_token_ids
        ):
            request.status = RequestStatus.FINISHED_STOPPED
            request.stop_reason = last_token
            return True
        if request.num_output_tokens >= request.max_tokens:
            request.status = RequestStatus.FINISHED_LENGTH_CAPPED
            return True
        if request.num_tokens >= self.max_model_len:
            request.status = RequestStatus.FINISHED_LENGTH_CAPPED
            return True
        return False

    def _free_request(self, request: Request) -> None:
        self.kv_cache_manager.free(request)
        self.finished_req_ids.add(request.request_id)
        # Keep the Request object in self.requests until the engine client
        # drains its final output, then the engine calls release().

    def release_request(self, req_id: str) -> None:
        self.requests.pop(req_id, None)

    def make_stats(self) -> SchedulerStats:
        return SchedulerStats(
            num_running_reqs=len(self.running),
            num_waiting_reqs=len(self.waiting),
            kv_cache_usage=self.kv_cache_manager.usage,
            prefix_cache_queries=self.prefix_cache_queries,
            prefix_cache_hits=self.prefix_cache_hits,
        )
