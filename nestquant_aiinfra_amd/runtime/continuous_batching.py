"""Slot lifecycle of the continuous-batching engine: which request sits in which of the fixed
decode slots, who waits, who is done.  Same names and behaviour as the reference's scheduler
(nestquant/runtime/continuous_batching.py:11-155); pure Python, no device state."""

from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass, field
from enum import Enum


class RequestStatus(str, Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"
    CANCELLED = "cancelled"


_TERMINAL = (RequestStatus.FINISHED, RequestStatus.CANCELLED)


@dataclass
class DecodeRequest:
    request_id: str
    prompt_token_ids: tuple[int, ...]
    max_new_tokens: int
    eos_token_id: int | None = None
    status: RequestStatus = RequestStatus.WAITING
    slot: int | None = None
    generated_token_ids: list[int] = field(default_factory=list)

    def __post_init__(self) -> None:
        if not self.request_id:
            raise ValueError("request_id must not be empty")
        if not self.prompt_token_ids:
            raise ValueError("prompt_token_ids must not be empty")
        if self.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be positive")

    @property
    def done(self) -> bool:
        """Whether the newest generated token ends the request."""
        if not self.generated_token_ids:
            return False
        if self.eos_token_id is not None and self.generated_token_ids[-1] == self.eos_token_id:
            return True
        return len(self.generated_token_ids) >= self.max_new_tokens

    @property
    def next_position(self) -> int:
        """Cache position the request's next input token is written at."""
        return len(self.prompt_token_ids) + max(len(self.generated_token_ids) - 1, 0)


class ContinuousBatchScheduler:
    """Waiting queue, slot table and registry of every request that has not been forgotten."""

    def __init__(self, capacity: int) -> None:
        if isinstance(capacity, bool) or not isinstance(capacity, int) or capacity < 1:
            raise ValueError("capacity must be a positive integer")
        self.capacity = capacity
        self._table: list[DecodeRequest | None] = [None] * capacity
        self._queue: OrderedDict[str, DecodeRequest] = OrderedDict()      # waiting, oldest first
        self._known: dict[str, DecodeRequest] = {}
        self._vacated: set[int] = set()                                   # freed since the last consume

    # -- views -------------------------------------------------------------------------------
    @property
    def slots(self) -> tuple[DecodeRequest | None, ...]:
        return tuple(self._table)

    @property
    def waiting(self) -> tuple[DecodeRequest, ...]:
        return tuple(self._queue.values())

    @property
    def running(self) -> tuple[DecodeRequest, ...]:
        return tuple(entry for entry in self._table if entry is not None)

    def active_mask(self) -> tuple[bool, ...]:
        return tuple(entry is not None for entry in self._table)

    def positions(self) -> tuple[int, ...]:
        return tuple(0 if entry is None else entry.next_position for entry in self._table)

    def pending_count(self) -> int:
        return len(self._queue)

    def free_slot_count(self) -> int:
        return self._table.count(None)

    def registered_count(self) -> int:
        return len(self._known)

    def get(self, request_id: str) -> DecodeRequest:
        return self._known[request_id]

    # -- transitions -------------------------------------------------------------------------
    def submit(self, request: DecodeRequest) -> None:
        if request.request_id in self._known:
            raise ValueError(f"duplicate request_id: {request.request_id}")
        self._known[request.request_id] = request
        self._queue[request.request_id] = request

    def admit(self, limit: int | None = None) -> tuple[DecodeRequest, ...]:
        """Move waiting requests, oldest first, into free slots, lowest slot first."""
        if limit is not None and (isinstance(limit, bool) or not isinstance(limit, int) or limit < 0):
            raise ValueError("limit must be a non-negative integer or None")
        free = [slot for slot, entry in enumerate(self._table) if entry is None]
        room = min(len(free), len(self._queue)) if limit is None else min(len(free), len(self._queue), limit)
        admitted = []
        for slot in free[:room]:
            _, request = self._queue.popitem(last=False)
            request.status, request.slot = RequestStatus.RUNNING, slot
            self._table[slot] = request
            self._vacated.discard(slot)
            admitted.append(request)
        return tuple(admitted)

    def record_tokens(self, tokens_by_slot: dict[int, int]) -> tuple[DecodeRequest, ...]:
        """Append one sampled token per slot; requests that hit EOS or their budget finish."""
        finished = []
        for slot, token in tokens_by_slot.items():
            if not 0 <= slot < self.capacity or self._table[slot] is None:
                raise ValueError(f"slot {slot} is not running")
            request = self._table[slot]
            request.generated_token_ids.append(int(token))
            if request.done:
                self._vacate(slot, RequestStatus.FINISHED)
                finished.append(request)
        return tuple(finished)

    def cancel(self, request_id: str) -> DecodeRequest:
        request = self._known[request_id]
        if request.status is RequestStatus.WAITING:
            del self._queue[request_id]
            request.status = RequestStatus.CANCELLED
        elif request.status is RequestStatus.RUNNING:
            self._vacate(request.slot, RequestStatus.CANCELLED)
        return request

    def consume_released_slots(self) -> tuple[int, ...]:
        released = tuple(sorted(self._vacated))
        self._vacated.clear()
        return released

    def forget_terminal(self, request_id: str) -> DecodeRequest:
        request = self._known[request_id]
        if request.status not in _TERMINAL:
            raise ValueError("only terminal requests can be forgotten")
        return self._known.pop(request_id)

    def _vacate(self, slot: int, status: RequestStatus) -> None:
        request = self._table[slot]
        if request is None:
            raise ValueError(f"slot {slot} is already free")
        request.status, request.slot = status, None
        self._table[slot] = None
        self._vacated.add(slot)
