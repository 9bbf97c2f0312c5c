"""Prefill-first batch scheduler with recompute preemption.

Queue behaviour follows nanovllm/engine/scheduler.py:9-98: waiting requests are
prefilled first (bounded by ``max_num_seqs`` and ``max_num_batched_tokens``; a
request that does not fit rotates to the back of the queue), otherwise every
running request decodes one token, evicting from the back of the running queue
when the block pool is exhausted.
"""

from collections import deque

from byox_vllm_amd.engine.block_manager import BlockManager, StateSlotManager
from byox_vllm_amd.engine.sequence import Sequence, SequenceStatus
from byox_vllm_amd.utils.logging import logger


class Scheduler:
    def __init__(self, config):
        self.max_num_seqs = config.max_num_seqs
        self.max_num_batched_tokens = config.max_num_batched_tokens
        self.eos = config.eos
        self.block_manager = BlockManager(config.num_kvcache_blocks, config.kvcache_block_size)
        self.waiting: deque[Sequence] = deque()
        self.running: deque[Sequence] = deque()
        # portioned stepping (models that set it: Config.portioned): a step is a list of (sequence, token count) pairs,
        # prompt pieces beside single decoded tokens; requests with a recurrent state also hold a state slot
        self.portioned = bool(getattr(config, "portioned", False))
        slots = getattr(config, "num_state_slots", 0)
        self.state_slots = StateSlotManager(slots) if slots > 0 else None
        # Quiet decode steps.  After a full pass over the running queue the scheduler knows for how many further steps
        # that pass would repeat itself exactly: as long as the queues do not change, every scheduled sequence grows by
        # one token per step, and none of them reaches a block boundary (length % block_size in {0, 1}: a block to
        # hash or a block to allocate), the pass changes nothing and returns the same batch.  Those steps return the
        # batch of the last pass without walking it (45 us per step for 128 sequences otherwise).
        self.quiet_steps = getattr(config, "scheduler_quiet_steps", True)
        self._quiet_left = 0              # further steps the last full pass stays valid for
        self._quiet_batch: list[Sequence] = []
        self._quiet_len = 0               # length the batch's first sequence must have at the next quiet step

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    def add(self, seq: Sequence) -> None:
        self.waiting.append(seq)
        self._quiet_left = 0

    def schedule(self) -> tuple[list[Sequence], bool]:
        batch = self._schedule_prefill()
        if batch:
            return batch, True
        return self._schedule_decode(), False

    def _schedule_prefill(self) -> list[Sequence]:
        batch: list[Sequence] = []
        budget = self.max_num_batched_tokens
        while self.waiting and len(batch) < self.max_num_seqs:
            seq = self.waiting[0]
            if len(seq) > budget:
                self.waiting.rotate(-1)
                break
            if not self.block_manager.can_allocate(seq):
                break
            self.block_manager.allocate(seq)
            budget -= len(seq) - seq.num_cached_tokens
            seq.status = SequenceStatus.RUNNING
            self.waiting.popleft()
            self.running.append(seq)
            batch.append(seq)
        if batch:
            self._quiet_left = 0
            logger.debug("[prefill] scheduled %s", batch)
        return batch

    def _schedule_decode(self) -> list[Sequence]:
        if self._quiet_left > 0 and len(self._quiet_batch[0]) == self._quiet_len:
            self._quiet_left -= 1
            self._quiet_len += 1
            return self._quiet_batch
        self._quiet_left = 0
        batch: list[Sequence] = []
        while self.running and len(batch) < self.max_num_seqs:
            seq = self.running.popleft()
            evicted_self = False
            while not self.block_manager.can_append(seq):
                if self.running:
                    self._preempt(self.running.pop())
                else:
                    self._preempt(seq)
                    evicted_self = True
                    break
            if not evicted_self:
                self.block_manager.may_append(seq)
                batch.append(seq)
        if batch:
            self.running.extendleft(reversed(batch))
            logger.debug("[decode] scheduled %s", batch)
            if self.quiet_steps:
                # steps until the first sequence of the batch has length % block_size == 0 (each step adds one token)
                bs = self.block_manager.block_size
                self._quiet_left = min((bs - 1 - r) if r else 0 for r in (len(seq) % bs for seq in batch))
                self._quiet_batch = batch
                self._quiet_len = len(batch[0]) + 1
        return batch

    def _preempt(self, seq: Sequence) -> None:
        logger.debug("preempting %s", seq)
        self._quiet_left = 0
        seq.status = SequenceStatus.WAITING
        self.block_manager.deallocate(seq)
        if self.state_slots is not None:
            self.state_slots.release(seq)
        self.waiting.appendleft(seq)

    # -- portioned stepping -----------------------------------------------------
    def commit(self, plan: list[tuple[Sequence, int]]) -> list[tuple[Sequence, int]]:
        """Make a step of (sequence, count) pairs runnable: admit sequences that are still waiting (state slot), grow
        their block tables to cover the tokens of this step.  The plan may come from schedule_portions (the engine's
        own policy) or from a caller that replays a fixed schedule; both run through here and through
        ModelRunner.run_portions.  Raises when the pools cannot hold the plan."""
        for seq, count in plan:
            assert 0 < count <= seq.num_tokens - seq.num_computed_tokens, f"{seq}: {count} tokens asked, " \
                f"{seq.num_tokens - seq.num_computed_tokens} left"
            if seq.status is SequenceStatus.WAITING:
                if self.state_slots is not None:
                    self.state_slots.allocate(seq)
                seq.status = SequenceStatus.RUNNING
                if seq in self.waiting:
                    self.waiting.remove(seq)
                self.running.append(seq)
            self.block_manager.extend(seq, seq.num_computed_tokens + count)
        return plan

    def schedule_portions(self) -> list[tuple[Sequence, int]]:
        """The engine's own policy for portioned stepping: every running request that is decoding gets its one token,
        then prompts (running ones first, then waiting ones in arrival order) get as large a piece as the step's token
        budget leaves.  Nothing is admitted that the block pool or the state slots cannot hold; when a decoding request
        cannot get its next block, the youngest running request is preempted (its prompt is recomputed later)."""
        budget = self.max_num_batched_tokens
        bm = self.block_manager
        plan: list[tuple[Sequence, int]] = []
        free = len(bm.free_block_ids)
        preempted = False
        for seq in list(self.running):
            if seq not in self.running:
                continue                       # preempted below
            left = seq.num_tokens - seq.num_computed_tokens
            count = min(left, budget)
            if count <= 0:
                continue
            need = bm.blocks_short(seq, seq.num_computed_tokens + count)
            while need > free and self.running[-1] is not seq:
                victim = self.running.pop()
                plan = [(s, c) for s, c in plan if s is not victim]
                self._preempt(victim)
                preempted = True
                free = len(bm.free_block_ids) - sum(bm.blocks_short(s, s.num_computed_tokens + c) for s, c in plan)
            if need > free:
                count = min(count, (len(seq.block_table) + free) * bm.block_size - seq.num_computed_tokens)
                if count <= 0:
                    continue
                need = bm.blocks_short(seq, seq.num_computed_tokens + count)
            plan.append((seq, count))
            budget -= count
            free -= need
        admitted = 0
        # a step that had to take pages away admits nobody: the preempted request would come straight back
        while not preempted and self.waiting and budget > 0 and len(self.running) + admitted < self.max_num_seqs:
            seq = self.waiting[0]
            if self.state_slots is not None and len(self.state_slots.free) <= admitted:
                break
            count = min(seq.num_tokens - seq.num_computed_tokens, budget, free * bm.block_size)
            if count <= 0:
                break
            self.waiting.popleft()             # commit() admits it: state slot, running queue, pages
            plan.append((seq, count))
            admitted += 1
            budget -= count
            free -= bm.blocks_short(seq, count)
        if not plan and (self.running or self.waiting):
            raise RuntimeError("no request can take a step: the block pool or the state slots are too small for the "
                               "oldest request alone (num_kvcache_blocks, num_state_slots)")
        return self.commit(plan)

    def advance(self, plan: list[tuple[Sequence, int]], token_ids: list[int | None]) -> list[Sequence]:
        """After a portioned step: count the tokens as computed; a request whose known tokens are all computed takes
        the token sampled for it (None: a replayed request that is fed its tokens from outside).  -> finished."""
        finished: list[Sequence] = []
        for (seq, count), token_id in zip(plan, token_ids):
            seq.num_computed_tokens += count
            if seq.num_computed_tokens < seq.num_tokens or token_id is None:
                continue
            seq.append_token(token_id)
            if (token_id == self.eos and not seq.ignore_eos) or seq.num_completion_tokens == seq.max_tokens:
                self.finish(seq)
                finished.append(seq)
        return finished

    def finish(self, seq: Sequence) -> None:
        """The request is over: its pages and its state slot go back to the pools."""
        seq.status = SequenceStatus.FINISHED
        self.block_manager.deallocate(seq)
        if self.state_slots is not None:
            self.state_slots.release(seq)
        if seq in self.running:
            self.running.remove(seq)
        if seq in self.waiting:
            self.waiting.remove(seq)
        self._quiet_left = 0

    def postprocess(self, seqs: list[Sequence], token_ids: list[int]) -> list[Sequence]:
        """Append the step's tokens; -> the sequences that finished with it (the reference returns nothing and has the
        engine look for them, llm_engine.py:52)."""
        eos = self.eos
        finished: list[Sequence] = []
        for seq, token_id in zip(seqs, token_ids):
            # Sequence.append_token and num_completion_tokens written out: this loop runs once per sequence and step
            seq.token_ids.append(token_id)
            seq.last_token = token_id
            seq.num_tokens = n = seq.num_tokens + 1
            if (token_id == eos and not seq.ignore_eos) or n - seq.num_prompt_tokens == seq.max_tokens:
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                self.running.remove(seq)
                self._quiet_left = 0
                finished.append(seq)
        return finished
