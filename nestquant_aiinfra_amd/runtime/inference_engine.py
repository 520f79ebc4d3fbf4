"""Continuous-batching engine over a fixed-capacity decode backend: admission, ragged prefill,
decode, sampling, slot release.  Same public surface as the reference's engine
(nestquant/runtime/inference_engine.py:14-285): RaggedDecodeBackend, AdmissionPolicy,
EngineStep, GreedyHostSampler, ContinuousBatchInferenceEngine.

What is added for a backend that samples on the device (BatchedNQKVLlamaRunner.decode_greedy):
with `decode_burst` > 1 a step in which nobody waits for a slot replays the captured decode
graph up to that many times before the host reads the chosen tokens once; requests that meet
their end-of-sequence token inside a burst are cut there.  A backend that says
`takes_slot_lists` is driven by slot lists instead of capacity-wide masks: a step then uploads
one row of tokens and positions per running request and reads nothing back before the launch,
and a prompt's logits are computed for its last token only."""

from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Protocol

import torch

from .continuous_batching import ContinuousBatchScheduler, DecodeRequest


class RaggedDecodeBackend(Protocol):
    batch_size: int
    max_cache_len: int
    device: torch.device

    def prefill(self, input_ids: torch.Tensor) -> torch.Tensor: ...
    def prefill_slots(self, input_ids: torch.Tensor, *, positions: torch.Tensor, write_mask: torch.Tensor,
                      valid_lengths: torch.Tensor) -> torch.Tensor: ...
    def capture(self, sample_token: torch.Tensor, *, positions: torch.Tensor, active_mask: torch.Tensor,
                valid_lengths: torch.Tensor) -> None: ...
    def decode(self, token: torch.Tensor, *, positions: torch.Tensor, active_mask: torch.Tensor,
               valid_lengths: torch.Tensor) -> torch.Tensor: ...
    def clear_slots(self, slot_mask: torch.Tensor) -> None: ...


@dataclass(frozen=True)
class EngineStep:
    admitted_request_ids: tuple[str, ...]
    generated_tokens: dict[str, int]
    finished_request_ids: tuple[str, ...]
    active_request_ids: tuple[str | None, ...]
    prefill_seconds: float
    decode_seconds: float


@dataclass(frozen=True)
class AdmissionPolicy:
    """Hold free slots for a few steps until a prompt microbatch worth a prefill has gathered."""

    min_prefill_batch: int = 4
    max_wait_steps: int = 2

    def __post_init__(self) -> None:
        for name, least in (("min_prefill_batch", 1), ("max_wait_steps", 0)):
            value = getattr(self, name)
            if isinstance(value, bool) or not isinstance(value, int) or value < least:
                raise ValueError(f"{name} must be an integer >= {least}")


class GreedyHostSampler:
    """Argmax over logits [requests, vocabulary], outside the captured graph."""

    def __call__(self, logits: torch.Tensor) -> torch.Tensor:
        if logits.ndim != 2:
            raise ValueError("sampler logits must have shape [requests, vocabulary]")
        return logits.argmax(dim=-1)


class ContinuousBatchInferenceEngine:
    """One `step()` = release finished slots, admit, prefill the admitted prompts as one ragged
    batch, decode the requests that were already running, sample, record."""

    def __init__(self, backend: RaggedDecodeBackend, *, pad_token_id: int = 0,
                 sampler: GreedyHostSampler | None = None, admission_policy: AdmissionPolicy | None = None,
                 decode_burst: int = 1) -> None:
        if isinstance(decode_burst, bool) or not isinstance(decode_burst, int) or decode_burst < 1:
            raise ValueError("decode_burst must be a positive integer")
        self.backend = backend
        self.capacity, self.max_cache_len, self.device = backend.batch_size, backend.max_cache_len, backend.device
        self.pad_token_id = int(pad_token_id)
        self.sampler = sampler or GreedyHostSampler()
        self.admission_policy = admission_policy or AdmissionPolicy()
        self.scheduler = ContinuousBatchScheduler(self.capacity)
        # bursts need the device sampler, which is greedy: any other sampler keeps one token per step
        self.decode_burst = decode_burst if (sampler is None and hasattr(backend, "decode_greedy")) else 1
        self._slot_lists = bool(getattr(backend, "takes_slot_lists", False))
        self._ready = False
        self._steps_taken = 0
        self._slots_idle_since: int | None = None

    # -- requests ----------------------------------------------------------------------------
    def submit(self, request: DecodeRequest) -> None:
        if len(request.prompt_token_ids) + request.max_new_tokens > self.max_cache_len:
            raise ValueError("prompt plus max_new_tokens exceeds the KV cache")
        self.scheduler.submit(request)

    def cancel(self, request_id: str) -> DecodeRequest:
        request = self.scheduler.cancel(request_id)
        self._release_vacated()
        return request

    def has_work(self) -> bool:
        return bool(self.scheduler.pending_count() or self.scheduler.running)

    def forget_terminal(self, request_id: str) -> DecodeRequest:
        return self.scheduler.forget_terminal(request_id)

    # -- set-up ------------------------------------------------------------------------------
    def _column(self, fill, dtype) -> torch.Tensor:
        return torch.full((self.capacity, 1), fill, dtype=dtype, device=self.device)

    @torch.inference_mode()
    def initialize(self) -> None:
        """Warm every slot with a one-token prompt, capture the decode graphs, free the slots."""
        if self._ready:
            return
        everyone = torch.ones(self.capacity, dtype=torch.bool, device=self.device)
        self.backend.prefill(self._column(self.pad_token_id, torch.long))
        self.backend.capture(self._column(self.pad_token_id, torch.long), positions=self._column(0, torch.long),
                             active_mask=self._column(True, torch.bool),
                             valid_lengths=torch.ones(self.capacity, dtype=torch.long, device=self.device))
        self.backend.clear_slots(everyone)
        self._ready = True

    def _release_vacated(self) -> None:
        vacated = self.scheduler.consume_released_slots()
        if vacated:
            mask = torch.zeros(self.capacity, dtype=torch.bool, device=self.device)
            mask[list(vacated)] = True
            self.backend.clear_slots(mask)

    def _valid_lengths(self) -> torch.Tensor:
        return torch.tensor([1 if entry is None else entry.next_position for entry in self.scheduler.slots],
                            dtype=torch.long, device=self.device)

    def _how_many_to_admit(self) -> int:
        waiting, free = self.scheduler.pending_count(), self.scheduler.free_slot_count()
        if not waiting or not free:
            self._slots_idle_since = None
            return 0
        batch = min(waiting, free)
        if not self.scheduler.running:                      # nothing to hold up: fill the slots now
            self._slots_idle_since = None
            return batch
        if self._slots_idle_since is None:
            self._slots_idle_since = self._steps_taken
        policy = self.admission_policy
        if batch >= policy.min_prefill_batch or self._steps_taken - self._slots_idle_since >= policy.max_wait_steps:
            self._slots_idle_since = None
            return batch
        return 0

    # -- the two halves of a step ------------------------------------------------------------
    def _prefill(self, admitted: tuple[DecodeRequest, ...]) -> tuple[dict[str, int], tuple[str, ...]]:
        if not admitted:
            return {}, ()
        width = max(len(request.prompt_token_ids) for request in admitted)
        if self._slot_lists:
            rows = [list(request.prompt_token_ids) + [self.pad_token_id] * (width - len(request.prompt_token_ids))
                    for request in admitted]
            logits = self.backend.prefill_slots(
                torch.tensor(rows, dtype=torch.long, device=self.device), slots=[request.slot for request in admitted],
                lengths=[len(request.prompt_token_ids) for request in admitted], last_token_logits=True)
            return self._record(admitted, [[token] for token in self.sampler(logits[:, 0]).tolist()])
        input_ids = torch.full((self.capacity, width), self.pad_token_id, dtype=torch.long, device=self.device)
        write_mask = torch.zeros((self.capacity, width), dtype=torch.bool, device=self.device)
        # every column of a row gets its own position, padding included
        positions = torch.arange(width, dtype=torch.long, device=self.device).repeat(self.capacity, 1)
        valid_lengths = self._valid_lengths()
        for request in admitted:
            prompt = torch.tensor(request.prompt_token_ids, dtype=torch.long, device=self.device)
            input_ids[request.slot, :prompt.numel()] = prompt
            write_mask[request.slot, :prompt.numel()] = True
            valid_lengths[request.slot] = prompt.numel()
        logits = self.backend.prefill_slots(input_ids, positions=positions, write_mask=write_mask,
                                            valid_lengths=valid_lengths)
        rows = torch.tensor([request.slot for request in admitted], device=self.device)
        last = torch.tensor([len(request.prompt_token_ids) - 1 for request in admitted], device=self.device)
        chosen = self.sampler(logits[rows, last]).tolist()
        return self._record(admitted, [[token] for token in chosen])

    def _record(self, requests, tokens_per_request) -> tuple[dict[str, int], tuple[str, ...]]:
        """Feed sampled tokens to the scheduler, one round per burst position; a request that finishes
        takes no further tokens of its burst."""
        newest: dict[str, int] = {}
        finished: list[str] = []
        for position in range(max(len(tokens) for tokens in tokens_per_request)):
            round_tokens = {request.slot: tokens[position] for request, tokens in zip(requests, tokens_per_request)
                            if request.slot is not None and position < len(tokens)}
            owners = {request.slot: request for request in requests if request.slot in round_tokens}
            for slot, token in round_tokens.items():
                newest[owners[slot].request_id] = int(token)
            finished.extend(request.request_id for request in self.scheduler.record_tokens(round_tokens))
        return newest, tuple(finished)

    def _decode(self, running: tuple[DecodeRequest, ...]) -> tuple[dict[str, int], tuple[str, ...]]:
        if not running:
            return {}, ()
        burst = 1
        if self.decode_burst > 1 and not self.scheduler.pending_count():
            budget = min(request.max_new_tokens - len(request.generated_token_ids) for request in running)
            burst = max(1, min(self.decode_burst, budget))
        if burst > 1:
            slots = [request.slot for request in running]
            tokens = torch.tensor([[request.generated_token_ids[-1]] for request in running], dtype=torch.long,
                                  device=self.device)
            positions = torch.tensor([[request.next_position] for request in running], dtype=torch.long,
                                     device=self.device)
            history = self.backend.decode_greedy(tokens, slots=slots, positions=positions, steps=burst).tolist()
            return self._record(running, [[history[step][row] for step in range(burst)] for row in range(len(running))])
        if self._slot_lists:
            tokens = torch.tensor([[request.generated_token_ids[-1]] for request in running], dtype=torch.long,
                                  device=self.device)
            positions = torch.tensor([[request.next_position] for request in running], dtype=torch.long,
                                     device=self.device)
            logits = self.backend.decode(tokens, slots=[request.slot for request in running], positions=positions)
            return self._record(running, [[value] for value in self.sampler(logits[:, -1]).tolist()])
        token = self._column(self.pad_token_id, torch.long)
        positions = self._column(0, torch.long)
        active = self._column(False, torch.bool)
        valid_lengths = self._valid_lengths()
        for request in running:
            token[request.slot, 0] = request.generated_token_ids[-1]
            positions[request.slot, 0] = request.next_position
            active[request.slot, 0] = True
            valid_lengths[request.slot] = request.next_position + 1
        logits = self.backend.decode(token, positions=positions, active_mask=active, valid_lengths=valid_lengths)
        rows = torch.tensor([request.slot for request in running], device=self.device)
        chosen = self.sampler(logits[rows, -1]).tolist()
        return self._record(running, [[value] for value in chosen])

    @torch.inference_mode()
    def step(self) -> EngineStep:
        if not self._ready:
            self.initialize()
        self._release_vacated()
        already_running = self.scheduler.running
        admitted = self.scheduler.admit(limit=self._how_many_to_admit())
        started = time.perf_counter()
        prefill_tokens, prefill_finished = self._prefill(admitted)
        between = time.perf_counter()
        decode_tokens, decode_finished = self._decode(already_running)
        ended = time.perf_counter()
        # a step that empties the workload must not leave the freed slots held until a next step
        self._release_vacated()
        self._steps_taken += 1
        return EngineStep(
            admitted_request_ids=tuple(request.request_id for request in admitted),
            generated_tokens={**decode_tokens, **prefill_tokens},
            finished_request_ids=decode_finished + prefill_finished,
            active_request_ids=tuple(None if entry is None else entry.request_id for entry in self.scheduler.slots),
            prefill_seconds=between - started, decode_seconds=ended - between)
