"""NQKV4 paged KV cache on the GPU: packed pages, the page pool, device-resident sequence
tables, the ragged writer and batched decode attention.

Mirrors the reference's surface for this path:
  PreparedNQKVPage / quantize_nqkv_page_cuda / dequantize_nqkv_page_triton   nestquant/runtime/nqkv_page.py:192-329, 494-537
  NQKVPageHandle / NQKVPagePool                                               nestquant/runtime/nqkv_pool.py:14-251
  BatchedNQKVMetadata                                                         nestquant/runtime/paged_nqkv_cache.py:25-95
  nqkv_decode_attention_batched_k1                                            nestquant/runtime/nqkv_attention_k1.py:763-942
The per-layer hot/cold cache object the kernels consume is NQKVHotColdCache (hot BF16 tails
plus the pool plus the tables; nestquant/runtime/nqkv_hot_cache.py:14-37).

Design difference, on purpose: lengths, page tables and hot-tail fill levels live on the
device and are advanced by one kernel per step (`BatchedNQKVCacheManager.begin_step`), and
every slot owns a fixed range of physical pages, so a decode step needs no host-side page
reservation, no host read of hot lengths and no separate page-boundary graph.
"""

from __future__ import annotations

import math
from collections import deque
from dataclasses import dataclass
from typing import Hashable, Sequence

import torch

from .. import _native
from .w4a4_linear import PreparedNQA4Activation, _beta_values, dequantize_rows_packed, quantize_rows_packed

PAGE_SIZE = 16


# --------------------------------------------------------------------------------------
# single pages
# --------------------------------------------------------------------------------------

@dataclass(frozen=True)
class PreparedNQKVPage:
    """One packed K/V page resident on the GPU (views into a pool or freshly encoded)."""

    key_code_payload: torch.Tensor
    key_beta_payload: torch.Tensor
    key_norms: torch.Tensor
    value_code_payload: torch.Tensor
    value_beta_payload: torch.Tensor
    value_norms: torch.Tensor
    key_beta_table: torch.Tensor
    value_beta_table: torch.Tensor
    page_size: int
    valid_tokens: int
    num_kv_heads: int
    head_dim: int
    q: int
    code_width: int
    beta_width: int
    output_dtype: torch.dtype

    @property
    def device(self) -> torch.device:
        return self.key_code_payload.device

    @property
    def payload_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (
            self.key_code_payload, self.key_beta_payload, self.key_norms,
            self.value_code_payload, self.value_beta_payload, self.value_norms))


def quantize_nqkv_page_cuda(key: torch.Tensor, value: torch.Tensor, *, page_size: int, q: int,
                            betas: Sequence[float] | None = None,
                            key_betas: Sequence[float] | None = None,
                            value_betas: Sequence[float] | None = None,
                            key_beta_table: torch.Tensor | None = None,
                            value_beta_table: torch.Tensor | None = None) -> PreparedNQKVPage:
    """Quantize an NHD K/V prefix [valid, kv_heads, head_dim] into one fixed-capacity page.

    Rows beyond the valid prefix are encoded zeros (norm 0), exactly as
    PackedNQKVPage.from_tensors does on the CPU (nestquant/core/kv_format.py:99-131).
    """
    if not isinstance(key, torch.Tensor) or not isinstance(value, torch.Tensor):
        raise TypeError("key and value must be tensors")
    if key.shape != value.shape or key.ndim != 3 or key.dtype != value.dtype:
        raise ValueError("key and value must share shape [tokens, kv_heads, head_dim] and dtype")
    if key.device.type != "cuda" or key.device != value.device:
        raise ValueError("key and value must share a CUDA device")
    valid, heads, dim = key.shape
    if not 1 <= valid <= page_size:
        raise ValueError("token count must be in [1, page_size]")
    if betas is not None:
        if key_betas is not None or value_betas is not None:
            raise ValueError("pass legacy betas or key_betas/value_betas, not both")
        key_values = value_values = _beta_values(betas)
    else:
        if key_betas is None or value_betas is None:
            raise ValueError("v2 requires both key_betas and value_betas")
        key_values, value_values = _beta_values(key_betas), _beta_values(value_betas)
    device = key.device
    if key_beta_table is None:
        key_beta_table = torch.tensor(key_values, device=device, dtype=torch.float32)
    if value_beta_table is None:
        value_beta_table = (key_beta_table if betas is not None
                            else torch.tensor(value_values, device=device, dtype=torch.float32))
    rows = page_size * heads
    streams = []
    for tensor, table in ((key, key_beta_table), (value, value_beta_table)):
        padded = torch.zeros((rows, dim), device=device, dtype=tensor.dtype)
        padded[: valid * heads].copy_(tensor.reshape(valid * heads, dim))
        streams.extend(quantize_rows_packed(padded, q=q, beta_table=table))
    return PreparedNQKVPage(*streams[0:3], *streams[3:6], key_beta_table, value_beta_table,
                            page_size, valid, heads, dim, q, 4, 2, key.dtype)


def dequantize_nqkv_page(page: PreparedNQKVPage, *, output_dtype: torch.dtype | None = None,
                         tile_blocks: int | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Decode a packed page back to its valid NHD prefix (float32 maths, then one cast)."""
    if not isinstance(page, PreparedNQKVPage):
        raise TypeError("page must be a PreparedNQKVPage")
    dtype = page.output_dtype if output_dtype is None else output_dtype
    rows = page.page_size * page.num_kv_heads
    shape = (page.page_size, page.num_kv_heads, page.head_dim)
    out = []
    for codes, ids, norms, table in (
            (page.key_code_payload, page.key_beta_payload, page.key_norms, page.key_beta_table),
            (page.value_code_payload, page.value_beta_payload, page.value_norms, page.value_beta_table)):
        full = dequantize_rows_packed(codes.contiguous(), ids.contiguous(), norms.contiguous(), table,
                                      rows=rows, features=page.head_dim, q=page.q, output_dtype=dtype)
        out.append(full.reshape(shape)[: page.valid_tokens])
    return out[0], out[1]


dequantize_nqkv_page_triton = dequantize_nqkv_page      # the reference's name for the same operator


# --------------------------------------------------------------------------------------
# page pool
# --------------------------------------------------------------------------------------

@dataclass(frozen=True)
class NQKVPageHandle:
    """Generation-checked ownership token for one physical page."""

    page_id: int
    generation: int


@dataclass
class _PageRecord:
    """Host-side state of one physical page."""

    generation: int = 0          # bumped on release: handles of an earlier owner stop matching
    owned: bool = False
    valid_tokens: int = 0        # 0 until a payload has been stored


def _positive(**values: int) -> None:
    for name, value in values.items():
        if isinstance(value, bool) or not isinstance(value, int) or value < 1:
            raise ValueError(f"{name} must be a positive integer")


class NQKVPagePool:
    """Preallocated SoA page storage (same tensors as the reference's pool,
    nestquant/runtime/nqkv_pool.py:94-110); the tensors never move, so kernels captured in a HIP
    graph keep valid addresses.  Ownership is host-side: one record per page, handles carry the
    page's generation and go stale when the page is released."""

    _STREAMS = ("key_codes", "key_betas", "key_norms", "value_codes", "value_betas", "value_norms")

    def __init__(self, *, capacity: int, page_size: int, num_kv_heads: int, head_dim: int, q: int,
                 betas: Sequence[float] | None = None, key_betas: Sequence[float] | None = None,
                 value_betas: Sequence[float] | None = None,
                 output_dtype: torch.dtype = torch.bfloat16, device: torch.device | str = "cuda",
                 hints: bool = False) -> None:
        _positive(capacity=capacity, page_size=page_size, num_kv_heads=num_kv_heads, head_dim=head_dim)
        if head_dim % 8:
            raise ValueError("head_dim must be divisible by 8")
        shared_table = betas is not None                    # format v1: one table for keys and values
        if shared_table and (key_betas is not None or value_betas is not None):
            raise ValueError("pass legacy betas or key_betas/value_betas, not both")
        if not shared_table and (key_betas is None or value_betas is None):
            raise ValueError("v2 requires both key_betas and value_betas")
        key_table = tuple(map(float, betas if shared_table else key_betas))
        value_table = key_table if shared_table else tuple(map(float, value_betas))
        if not key_table or not value_table:
            raise ValueError("beta tables must be nonempty")
        where = torch.device(device)
        if where.type != "cuda" or not torch.cuda.is_available():
            raise ValueError("NQKVPagePool requires an available CUDA device")
        if where.index is None:
            where = torch.device("cuda", torch.cuda.current_device())

        self.capacity, self.page_size, self.num_kv_heads, self.head_dim, self.q = (
            capacity, page_size, num_kv_heads, head_dim, q)
        self.betas, self.value_beta_values = key_table, value_table
        self.format_version = 1 if shared_table else 2
        self.output_dtype, self.device = output_dtype, where
        self.code_width, self.beta_width = 4, 2
        rows = page_size * num_kv_heads                     # one row per (token, head)
        self._stream_shapes = {"codes": (rows * head_dim // 2, torch.uint8), "betas": (rows * head_dim // 32, torch.uint8),
                               "norms": (rows, torch.float32)}
        for side in ("key", "value"):
            for kind, (width, dtype) in self._stream_shapes.items():
                setattr(self, f"{side}_{kind}", torch.zeros((capacity, width), dtype=dtype, device=where))
        # Decode hints (not part of the reference's page format): four bits per block beside the six
        # streams, written by the kernels that pack a page and read by the attention kernels, which
        # then skip the lattice searches of the undithered decode.  Same decoded values bit for bit.
        self.key_hints = self.value_hints = None
        if hints:
            if q != 14 or (rows * head_dim // 8) % 2:
                raise ValueError("decode hints need q = 14 and an even number of blocks per page")
            self.key_hints = torch.zeros((capacity, rows * head_dim // 16), dtype=torch.uint8, device=where)
            self.value_hints = torch.zeros_like(self.key_hints)
        self.beta_table = torch.tensor(key_table, dtype=torch.float32, device=where)
        self.value_beta_table = self.beta_table if shared_table else torch.tensor(value_table, dtype=torch.float32,
                                                                                  device=where)
        self._pages = [_PageRecord() for _ in range(capacity)]
        self._unowned = deque(range(capacity))              # lowest page first

    # -- sizes -------------------------------------------------------------------------------
    @property
    def free_pages(self) -> int:
        return len(self._unowned)

    @property
    def allocated_pages(self) -> int:
        return self.capacity - len(self._unowned)

    @property
    def page_payload_bytes(self) -> int:
        return 2 * sum(width * dtype.itemsize for width, dtype in self._stream_shapes.values())

    @property
    def resident_bytes(self) -> int:
        held = [getattr(self, name) for name in self._STREAMS] + [self.beta_table]
        if self.value_beta_table is not self.beta_table:
            held.append(self.value_beta_table)
        if self.key_hints is not None:
            held += [self.key_hints, self.value_hints]
        return sum(tensor.numel() * tensor.element_size() for tensor in held)

    # -- ownership ---------------------------------------------------------------------------
    def allocate(self) -> NQKVPageHandle:
        if not self._unowned:
            raise RuntimeError("NQKV page pool is exhausted")
        page_id = self._unowned.popleft()
        record = self._pages[page_id]
        record.owned, record.valid_tokens = True, 0
        return NQKVPageHandle(page_id, record.generation)

    def release(self, handle: NQKVPageHandle) -> None:
        page_id = self._owned_page(handle)
        record = self._pages[page_id]
        record.owned, record.valid_tokens = False, 0
        record.generation += 1
        self._unowned.appendleft(page_id)                   # reused next, while it may still be cached

    def _owned_page(self, handle: NQKVPageHandle) -> int:
        if not isinstance(handle, NQKVPageHandle):
            raise TypeError("handle must be an NQKVPageHandle")
        if not 0 <= handle.page_id < self.capacity:
            raise ValueError("NQKV page ID is outside pool capacity")
        record = self._pages[handle.page_id]
        if not record.owned or record.generation != handle.generation:
            raise RuntimeError("stale or released NQKV page handle")
        return handle.page_id

    # -- payloads ----------------------------------------------------------------------------
    def store_prepared(self, handle: NQKVPageHandle, page: PreparedNQKVPage) -> None:
        """Copy a GPU-produced packed page into its fixed physical slot."""
        page_id = self._owned_page(handle)
        if not isinstance(page, PreparedNQKVPage):
            raise TypeError("page must be a PreparedNQKVPage")
        geometry = (self.page_size, self.num_kv_heads, self.head_dim, self.q, self.device)
        if (page.page_size, page.num_kv_heads, page.head_dim, page.q, page.device) != geometry:
            raise ValueError("prepared NQKV page configuration does not match the pool")
        if not (torch.equal(page.key_beta_table, self.beta_table)
                and torch.equal(page.value_beta_table, self.value_beta_table)):
            raise ValueError("prepared NQKV beta tables do not match the pool")
        incoming = (page.key_code_payload, page.key_beta_payload, page.key_norms,
                    page.value_code_payload, page.value_beta_payload, page.value_norms)
        slots = [getattr(self, name)[page_id] for name in self._STREAMS]
        if any(slot.numel() != stream.numel() for slot, stream in zip(slots, incoming)):
            raise ValueError("prepared NQKV payload sizes do not match the pool")
        for slot, stream in zip(slots, incoming):
            slot.copy_(stream)
        if self.key_hints is not None:                   # a page from elsewhere: its hints from its code words
            lib, stream_handle = _native.library(), _native.stream_handle(self.device)
            for codes, hints in ((self.key_codes, self.key_hints), (self.value_codes, self.value_hints)):
                _native.check(lib.nq_nqkv_page_hints(codes[page_id].data_ptr(), codes.shape[1] // 4,
                                                     hints[page_id].data_ptr(), stream_handle))
        self._pages[page_id].valid_tokens = page.valid_tokens

    def store(self, handle: NQKVPageHandle, page) -> None:
        """Copy a host container (core.kv_format.PackedNQKVPage) into the page's physical slot."""
        if not hasattr(page, "to_prepared"):
            raise TypeError("page must be a PackedNQKVPage")
        self.store_prepared(handle, page.to_prepared(self.device))

    def mark_graph_stored(self, handle: NQKVPageHandle, *, valid_tokens: int) -> None:
        """Record that a kernel (not store_prepared) has filled the page."""
        page_id = self._owned_page(handle)
        if not 1 <= valid_tokens <= self.page_size:
            raise ValueError("valid_tokens must be in [1, page_size]")
        self._pages[page_id].valid_tokens = valid_tokens

    def prepared(self, handle: NQKVPageHandle) -> PreparedNQKVPage:
        page_id = self._owned_page(handle)
        tokens = self._pages[page_id].valid_tokens
        if not tokens:
            raise RuntimeError("NQKV page has not been stored")
        return self.page_view(page_id, tokens)

    def hint_pointers(self) -> tuple[int | None, int | None]:
        """The two hint streams as the C ABI takes them (None, None without hints)."""
        if self.key_hints is None:
            return None, None
        return self.key_hints.data_ptr(), self.value_hints.data_ptr()

    def page_view(self, page_id: int, valid_tokens: int) -> PreparedNQKVPage:
        return PreparedNQKVPage(
            *(getattr(self, name)[page_id] for name in self._STREAMS), self.beta_table, self.value_beta_table,
            self.page_size, valid_tokens, self.num_kv_heads, self.head_dim, self.q, self.code_width, self.beta_width,
            self.output_dtype)


# --------------------------------------------------------------------------------------
# device-resident sequence tables
# --------------------------------------------------------------------------------------

@dataclass(frozen=True)
class BatchedNQKVMetadata:
    """Fixed-address GPU metadata consumed by the batched paged NQKV kernels."""

    slot_ids: torch.Tensor
    page_indptr: torch.Tensor
    page_indices: torch.Tensor
    page_counts: torch.Tensor
    last_page_lens: torch.Tensor
    hot_lengths: torch.Tensor
    sequence_lengths: torch.Tensor
    active_mask: torch.Tensor
    # the four per-slot counters as rows of one int32 [4, capacity] tensor (None when they were
    # allocated one by one): a run of slots is then reset with one fill instead of four
    counters: torch.Tensor | None = None

    @classmethod
    def create(cls, *, capacity: int, max_pages_per_sequence: int,
               device: torch.device | str) -> "BatchedNQKVMetadata":
        for name, value in (("capacity", capacity), ("max_pages_per_sequence", max_pages_per_sequence)):
            if isinstance(value, bool) or not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be a positive integer")
        target = torch.device(device)
        counters = torch.zeros((4, capacity), dtype=torch.int32, device=target)
        return cls(
            slot_ids=torch.arange(capacity, dtype=torch.int32, device=target),
            page_indptr=torch.arange(0, (capacity + 1) * max_pages_per_sequence, max_pages_per_sequence,
                                     dtype=torch.int32, device=target),
            page_indices=torch.full((capacity, max_pages_per_sequence), -1, dtype=torch.int32, device=target),
            page_counts=counters[0], last_page_lens=counters[1], hot_lengths=counters[2], sequence_lengths=counters[3],
            active_mask=torch.zeros(capacity, dtype=torch.bool, device=target), counters=counters,
        )

    def pointers(self) -> tuple[int, ...]:
        return tuple(t.data_ptr() for t in (
            self.slot_ids, self.page_indptr, self.page_indices, self.page_counts, self.last_page_lens,
            self.hot_lengths, self.sequence_lengths, self.active_mask))


class NQKVHotColdCache:
    """One layer's cache: packed cold pages in a pool, a BF16 hot tail per slot, and the
    (possibly shared) device tables that say how much of each is valid.

    Two ways to build one.  `NQKVHotColdCache(pool, metadata, max_sequences=, max_pages_per_sequence=)`
    is the flat form the batched manager uses: slots own fixed pages and the tables are shared between
    layers.  `NQKVHotColdCache(cold_cache)` over a PagedNQKVCache is the reference's form
    (nestquant/runtime/nqkv_hot_cache.py:14-37): sequences are registered by id, `append` takes pages
    from the pool as tails fill, and `hot_view` / `materialize` / `total_tokens` read one sequence."""

    def __init__(self, pool, metadata: BatchedNQKVMetadata | None = None, *, max_sequences: int | None = None,
                 max_pages_per_sequence: int | None = None) -> None:
        self._logical = None
        if not isinstance(pool, NQKVPagePool):
            logical = pool
            if not all(hasattr(logical, name) for name in ("pool", "metadata", "reserve_page", "commit_graph_page")):
                raise TypeError("cold_cache must be a PagedNQKVCache")
            if metadata is not None or max_sequences is not None or max_pages_per_sequence is not None:
                raise ValueError("a cache over a PagedNQKVCache takes its tables and sizes from it")
            self._logical = logical
            pool, metadata = logical.pool, logical.metadata
            max_sequences, max_pages_per_sequence = logical.max_sequences, logical.max_pages_per_sequence
        elif metadata is None or max_sequences is None or max_pages_per_sequence is None:
            raise ValueError("the flat form needs metadata, max_sequences and max_pages_per_sequence")
        self.pool, self.metadata = pool, metadata
        self.max_sequences, self.max_pages_per_sequence = max_sequences, max_pages_per_sequence
        shape = (max_sequences, pool.page_size, pool.num_kv_heads, pool.head_dim)
        self.hot_keys = torch.zeros(shape, device=pool.device, dtype=torch.bfloat16)
        self.hot_values = torch.zeros_like(self.hot_keys)
        self.hot_lengths = metadata.hot_lengths
        self._hot_tokens = [0] * max_sequences          # host mirror of the tails (sequence form only)

    @property
    def cold_cache(self):
        """The PagedNQKVCache underneath, or the cache itself in the flat form."""
        return self if self._logical is None else self._logical

    # -- one sequence at a time (over a PagedNQKVCache) --------------------------------------------
    def _sequences(self):
        if self._logical is None:
            raise RuntimeError("this cache is driven by slot through its manager: it holds no sequence ids")
        return self._logical

    def register(self, sequence_id: Hashable, *, slot: int | None = None) -> int:
        slot = self._sequences().register(sequence_id, slot=slot)
        self._hot_tokens[slot] = 0
        return slot

    def release(self, sequence_id: Hashable) -> None:
        logical = self._sequences()
        slot = logical.slot(sequence_id)
        logical.release(sequence_id)
        self._hot_tokens[slot] = 0

    def hot_length(self, slot: int) -> int:
        self._sequences().sequence_id(slot)
        return self._hot_tokens[slot]

    def total_tokens(self, sequence_id: Hashable) -> int:
        logical = self._sequences()
        return logical.total_tokens(sequence_id) + self._hot_tokens[logical.slot(sequence_id)]

    def hot_view(self, sequence_id: Hashable) -> tuple[torch.Tensor, torch.Tensor]:
        slot = self._sequences().slot(sequence_id)
        held = self._hot_tokens[slot]
        return self.hot_keys[slot, :held], self.hot_values[slot, :held]

    def append(self, sequence_id: Hashable, key: torch.Tensor, value: torch.Tensor) -> None:
        """Append key / value BF16 [tokens, kv_heads, head_dim] (keys already rotated) to one sequence.
        The pages this append completes are reserved from the pool and mapped into the sequence's page
        table first; the writer kernel then fills the tail and encodes those pages in one launch."""
        logical = self._sequences()
        slot = logical.slot(sequence_id)
        pool = self.pool
        if (not isinstance(key, torch.Tensor) or key.ndim != 3 or key.shape != value.shape
                or tuple(key.shape[1:]) != (pool.num_kv_heads, pool.head_dim)):
            raise ValueError("key and value must share shape [tokens, kv_heads, head_dim]")
        if key.dtype != torch.bfloat16 or value.dtype != torch.bfloat16 or key.device != pool.device:
            raise ValueError("key and value must be BF16 on the cache device")
        tokens = key.shape[0]
        if tokens < 1:
            return
        held = self._hot_tokens[slot]
        if logical.total_tokens(sequence_id) != len(logical.handles(sequence_id)) * pool.page_size:
            raise RuntimeError("a sequence whose newest page is partial takes whole pages only")
        if logical.total_tokens(sequence_id) + held + tokens > self.max_pages_per_sequence * pool.page_size:
            raise RuntimeError("sequence exceeds max_pages_per_sequence")
        completes = (held + tokens) // pool.page_size
        first_ordinal = len(logical.handles(sequence_id))
        handles = []
        try:
            for _ in range(completes):
                handles.append(logical.reserve_page(sequence_id))
        except Exception:
            for handle in handles:
                logical.cancel_reserved_page(sequence_id, handle)
            raise
        meta = self.metadata
        if handles:
            meta.page_indices[slot, first_ordinal:first_ordinal + completes] = torch.tensor(
                [handle.page_id for handle in handles], dtype=torch.int32, device=pool.device)
        slot_ids = torch.tensor([slot], dtype=torch.int32, device=pool.device)
        active = torch.ones(1, dtype=torch.bool, device=pool.device)
        lib, stream = _native.library(), _native.stream_handle(pool.device)
        _native.check(lib.nq_nqkv_advance(
            slot_ids.data_ptr(), active.data_ptr(), None, tokens, 1, self.max_sequences, pool.page_size,
            self.max_pages_per_sequence * pool.page_size, meta.sequence_lengths.data_ptr(), meta.page_counts.data_ptr(),
            meta.last_page_lens.data_ptr(), meta.hot_lengths.data_ptr(), stream))
        key, value = key.contiguous(), value.contiguous()
        _native.check(lib.nq_nqkv_write(
            key.data_ptr(), value.data_ptr(), _native.dtype_tag(key.dtype), slot_ids.data_ptr(), active.data_ptr(),
            None, tokens, meta.sequence_lengths.data_ptr(), meta.page_indices.data_ptr(),
            pool.key_codes.data_ptr(), pool.key_betas.data_ptr(), pool.key_norms.data_ptr(),
            pool.value_codes.data_ptr(), pool.value_betas.data_ptr(), pool.value_norms.data_ptr(),
            pool.beta_table.data_ptr(), pool.beta_table.numel(), pool.value_beta_table.data_ptr(),
            pool.value_beta_table.numel(), self.hot_keys.data_ptr(), self.hot_values.data_ptr(),
            1, tokens, self.max_sequences, self.max_pages_per_sequence, pool.num_kv_heads, pool.head_dim,
            pool.page_size, 0, None, None, *pool.hint_pointers(), stream))
        for handle in handles:
            logical.commit_graph_page(sequence_id, handle)
        self._hot_tokens[slot] = (held + tokens) % pool.page_size

    def materialize(self, sequence_id: Hashable) -> tuple[torch.Tensor, torch.Tensor]:
        """The sequence as BF16 [tokens, kv_heads, head_dim]: its packed pages decoded, then the tail."""
        logical = self._sequences()
        keys, values = [], []
        for handle in logical.handles(sequence_id):
            key, value = dequantize_nqkv_page(self.pool.prepared(handle))
            keys.append(key)
            values.append(value)
        hot_key, hot_value = self.hot_view(sequence_id)
        if hot_key.shape[0]:
            keys.append(hot_key)
            values.append(hot_value)
        if not keys:
            empty = torch.empty((0, self.pool.num_kv_heads, self.pool.head_dim), device=self.pool.device,
                                dtype=self.pool.output_dtype)
            return empty, empty.clone()
        return torch.cat(keys), torch.cat(values)


@dataclass
class BatchedNQKVAttentionWorkspace:
    """Scratch for the two-stage attention (chunk maxima, sums and numerators) + output."""

    buffer: torch.Tensor
    output: torch.Tensor
    batch_size: int
    max_pages: int
    query_heads: int
    head_dim: int

    @classmethod
    def create(cls, cache: NQKVHotColdCache, *, batch_size: int, query_heads: int,
               output_dtype: torch.dtype) -> "BatchedNQKVAttentionWorkspace":
        pool = cache.pool
        need = _native.library().nq_nqkv_attention_workspace_bytes(
            batch_size, query_heads, pool.head_dim, cache.max_pages_per_sequence)
        return cls(torch.empty(need, dtype=torch.uint8, device=pool.device),
                   torch.empty((batch_size, query_heads, pool.head_dim), dtype=output_dtype, device=pool.device),
                   batch_size, cache.max_pages_per_sequence, query_heads, pool.head_dim)


def launch_nqkv_decode_attention(query: torch.Tensor, cache: NQKVHotColdCache, *, slot_ids: torch.Tensor,
                                 active_mask: torch.Tensor, attention_scale: float,
                                 workspace: BatchedNQKVAttentionWorkspace,
                                 rotate_query: bool = False,
                                 rope: tuple[torch.Tensor, torch.Tensor] | None = None,
                                 merge: bool = True) -> torch.Tensor | None:
    """Graph-safe launch: no host reads, no allocation; writes workspace.output.  `rope`:
    BF16 (cos, sin) [batch, head_dim] applied to the query inside the kernel.  With `merge`
    false only the first stage runs and the per-chunk results stay in workspace.buffer for
    attention_output_stage (returns None)."""
    pool, meta = cache.pool, cache.metadata
    batch, heads, dim = query.shape
    if not query.is_contiguous() or query.data_ptr() % 16:
        raise ValueError("query must be contiguous and 16-byte aligned (call .contiguous() on a sliced view)")
    if rope is not None and any(not t.is_contiguous() or t.dtype != torch.bfloat16 for t in rope):
        raise ValueError("rope must be a pair of contiguous BF16 tables")
    _native.check(_native.library().nq_nqkv_attention_decode(
        query.data_ptr(), _native.dtype_tag(query.dtype),
        pool.key_codes.data_ptr(), pool.key_betas.data_ptr(), pool.key_norms.data_ptr(),
        pool.value_codes.data_ptr(), pool.value_betas.data_ptr(), pool.value_norms.data_ptr(),
        pool.beta_table.data_ptr(), pool.value_beta_table.data_ptr(),
        meta.page_indices.data_ptr(), meta.page_counts.data_ptr(), meta.last_page_lens.data_ptr(),
        meta.hot_lengths.data_ptr(), meta.active_mask.data_ptr(),
        cache.hot_keys.data_ptr(), cache.hot_values.data_ptr(), slot_ids.data_ptr(), active_mask.data_ptr(),
        batch, cache.max_sequences, cache.max_pages_per_sequence, heads, pool.num_kv_heads, dim, pool.page_size,
        attention_scale, int(rotate_query), None if rope is None else rope[0].data_ptr(),
        None if rope is None else rope[1].data_ptr(), workspace.output.data_ptr() if merge else None,
        workspace.buffer.data_ptr(), workspace.buffer.numel(), *pool.hint_pointers(),
        _native.stream_handle(query.device)))
    return workspace.output if merge else None


def attention_output_stage(workspace: BatchedNQKVAttentionWorkspace, *, q: int = 14,
                           beta_table: torch.Tensor | None = None, hadamard: bool = True, encode: bool = True,
                           want_staged: bool = False):
    """Second stage of launch_nqkv_decode_attention(..., merge=False) fused with the input stage
    of the Linear that consumes the attention output: merges the per-chunk results into BF16 rows
    [batch, query_heads * head_dim] and (with `encode`) rotates, encodes and packs them in the
    same launch.  Returns (packed activation or None, merged rows when `want_staged`)."""
    device = workspace.buffer.device
    batch, n = workspace.batch_size, workspace.query_heads * workspace.head_dim
    staged = torch.empty((batch, n), dtype=torch.bfloat16, device=device) if want_staged else None
    codes = beta_ids = norms = decoded = None
    if encode:
        if beta_table is None or q != 14 or beta_table.numel() != 4:
            raise ValueError("encoding needs q = 14 and a table of four betas")
        codes = torch.empty(batch * n // 2, dtype=torch.uint8, device=device)
        beta_ids = torch.empty(batch * n // 32, dtype=torch.uint8, device=device)
        norms = torch.empty(batch, dtype=torch.float32, device=device)
        decoded = torch.empty((batch, n), dtype=torch.bfloat16, device=device)
    elif not want_staged:
        raise ValueError("nothing to produce")

    def ptr(tensor):
        return None if tensor is None else tensor.data_ptr()

    lib = _native.library()
    parts = lib.nq_nqkv_attention_parts(batch, workspace.max_pages)
    _native.check(lib.nq_attention_output_stage(
        workspace.buffer.data_ptr(), batch, workspace.query_heads, workspace.head_dim, parts, ptr(staged), q,
        ptr(beta_table), 0 if beta_table is None else beta_table.numel(), int(hadamard), ptr(codes), ptr(beta_ids),
        ptr(norms), ptr(decoded), _native.stream_handle(device)))
    activation = None
    if encode:
        activation = PreparedNQA4Activation(
            code_payload=codes, beta_payload=beta_ids, row_norms=norms, beta_table=beta_table,
            original_shape=(batch, n), q=q, code_width=4, beta_width=2, output_dtype=torch.bfloat16,
            decoded=decoded)
    return activation, staged


def nqkv_decode_attention_batched_k1(query: torch.Tensor, cache: NQKVHotColdCache, *, slot_ids: torch.Tensor,
                                     active_mask: torch.Tensor, scale: float | None = None,
                                     workspace: BatchedNQKVAttentionWorkspace | None = None,
                                     rotate_query: bool = False) -> torch.Tensor:
    """Fused packed-cold plus BF16-hot decode attention for a ragged batch.

    query [batch, query_heads, head_dim]; slot_ids int32 [batch]; active_mask bool [batch].
    Unlike the reference there is no page-count limit and no host-side validation pass over
    slot contents (rows with nothing to attend to return zeros).
    """
    if not isinstance(query, torch.Tensor) or query.ndim != 3:
        raise ValueError("query must have shape [batch, query_heads, head_dim]")
    if not isinstance(slot_ids, torch.Tensor) or not isinstance(active_mask, torch.Tensor):
        raise TypeError("slot_ids and active_mask must be tensors")
    pool = cache.pool
    batch, heads, dim = query.shape
    if query.device != pool.device or dim != pool.head_dim:
        raise ValueError("query must match the cache CUDA device and head_dim")
    if heads < 1 or heads % pool.num_kv_heads:
        raise ValueError("query_heads must be a positive multiple of num_kv_heads")
    if slot_ids.dtype != torch.int32 or tuple(slot_ids.shape) != (batch,):
        raise ValueError("slot_ids must be int32 with shape [batch]")
    if active_mask.dtype != torch.bool or tuple(active_mask.shape) != (batch,):
        raise ValueError("active_mask must be bool with shape [batch]")
    if slot_ids.device != pool.device or active_mask.device != pool.device:
        raise ValueError("slot_ids and active_mask must be on the cache device")
    if workspace is None:
        workspace = BatchedNQKVAttentionWorkspace.create(cache, batch_size=batch, query_heads=heads,
                                                         output_dtype=query.dtype)
    if (workspace.batch_size, workspace.max_pages, workspace.query_heads, workspace.head_dim,
            workspace.output.dtype) != (batch, cache.max_pages_per_sequence, heads, dim, query.dtype):
        raise ValueError("batched workspace configuration does not match query and cache")
    attention_scale = 1.0 / math.sqrt(dim) if scale is None else float(scale)
    if not math.isfinite(attention_scale):
        raise ValueError("scale must be finite")
    return launch_nqkv_decode_attention(query.contiguous(), cache, slot_ids=slot_ids, active_mask=active_mask,
                                        attention_scale=attention_scale, workspace=workspace,
                                        rotate_query=rotate_query)


def nqkv_prefill_attention(query: torch.Tensor, cache: NQKVHotColdCache, *, slot_ids: torch.Tensor,
                           active_mask: torch.Tensor, counts: torch.Tensor | None = None, uniform_count: int | None = None,
                           scale: float | None = None, split_context: bool = True) -> torch.Tensor:
    """Causal attention of a chunk of new tokens over the packed cache, after the chunk was
    written: query BF16 [batch, tokens, query_heads, head_dim] (rotated like the stored keys);
    row r holds counts[r] (or uniform_count) new tokens that end at the slot's sequence length.
    Returns BF16 [batch, tokens, query_heads, head_dim]; padding tokens give zeros.  `split_context`
    lets the library split long page tables over more workgroups (partial results in a scratch buffer,
    merged by a second launch); without it one workgroup walks a row's whole context."""
    if not isinstance(query, torch.Tensor) or query.ndim != 4 or query.dtype != torch.bfloat16:
        raise ValueError("query must be BF16 [batch, tokens, query_heads, head_dim]")
    pool, meta = cache.pool, cache.metadata
    batch, tokens, heads, dim = query.shape
    if query.device != pool.device or dim != pool.head_dim:
        raise ValueError("query must match the cache CUDA device and head_dim")
    if heads < 1 or heads % pool.num_kv_heads:
        raise ValueError("query_heads must be a positive multiple of num_kv_heads")
    if (counts is None) == (uniform_count is None):
        raise ValueError("give either counts or uniform_count")
    if slot_ids.dtype != torch.int32 or slot_ids.numel() < batch or active_mask.dtype != torch.bool:
        raise ValueError("slot_ids must be int32 and active_mask bool, one entry per row")
    if counts is not None and (counts.dtype != torch.int32 or counts.numel() < batch):
        raise ValueError("counts must be int32 with one entry per row")
    attention_scale = 1.0 / math.sqrt(dim) if scale is None else float(scale)
    query = query.contiguous()
    out = torch.empty_like(query)
    lib = _native.library()
    # room for the partial results of a split context (long tables, few rows): the kernel then
    # spreads every row over the chip in proportion to its context
    need = 0 if not split_context else lib.nq_nqkv_attention_prefill_workspace_bytes(
        batch, tokens, cache.max_pages_per_sequence, heads, pool.num_kv_heads)
    workspace = torch.empty(need, dtype=torch.uint8, device=query.device) if need else None
    _native.check(lib.nq_nqkv_attention_prefill(
        query.data_ptr(), pool.key_codes.data_ptr(), pool.key_betas.data_ptr(), pool.key_norms.data_ptr(),
        pool.value_codes.data_ptr(), pool.value_betas.data_ptr(), pool.value_norms.data_ptr(),
        pool.beta_table.data_ptr(), pool.value_beta_table.data_ptr(), meta.page_indices.data_ptr(),
        meta.page_counts.data_ptr(), meta.last_page_lens.data_ptr(), meta.hot_lengths.data_ptr(),
        meta.sequence_lengths.data_ptr(), cache.hot_keys.data_ptr(), cache.hot_values.data_ptr(),
        slot_ids.data_ptr(), active_mask.data_ptr(), None if counts is None else counts.data_ptr(),
        0 if uniform_count is None else int(uniform_count), batch, tokens, cache.max_sequences,
        cache.max_pages_per_sequence, heads, pool.num_kv_heads, dim, pool.page_size, attention_scale,
        out.data_ptr(), None if workspace is None else workspace.data_ptr(), need, *pool.hint_pointers(),
        _native.stream_handle(query.device)))
    return out


# --------------------------------------------------------------------------------------
# single-cache writer under the reference's names
# --------------------------------------------------------------------------------------

def _check_hot_k1_inputs(key: torch.Tensor, value: torch.Tensor, cache: NQKVHotColdCache,
                         slot_ids: torch.Tensor, active_mask: torch.Tensor) -> int:
    if not isinstance(cache, NQKVHotColdCache):
        raise TypeError("cache must be an NQKVHotColdCache")
    pool = cache.pool
    if not isinstance(key, torch.Tensor) or not isinstance(value, torch.Tensor):
        raise TypeError("key and value must be tensors")
    if key.ndim != 3 or key.shape != value.shape or tuple(key.shape[1:]) != (pool.num_kv_heads, pool.head_dim):
        raise ValueError("key and value must have shape [batch, kv_heads, head_dim]")
    batch = key.shape[0]
    if not 1 <= batch <= cache.max_sequences:
        raise ValueError("batch must be within cache capacity")
    if key.dtype != torch.bfloat16 or value.dtype != torch.bfloat16:
        raise ValueError("key and value must be BF16 like the hot tails")
    if slot_ids.dtype != torch.int32 or tuple(slot_ids.shape) != (batch,):
        raise ValueError("slot_ids must be int32 with shape [batch]")
    if active_mask.dtype != torch.bool or tuple(active_mask.shape) != (batch,):
        raise ValueError("active_mask must be bool with shape [batch]")
    if any(t.device != pool.device for t in (key, value, slot_ids, active_mask)):
        raise ValueError("append inputs must be on the cache device")
    if not all(t.is_contiguous() for t in (key, value, slot_ids, active_mask)):
        raise RuntimeError("append inputs must be contiguous")
    return batch


def _launch_append_hot_k1_graph_safe(key: torch.Tensor, value: torch.Tensor, cache: NQKVHotColdCache, *,
                                     slot_ids: torch.Tensor, active_mask: torch.Tensor) -> None:
    """Fixed-address GPU work only: one table update and one writer launch, no host reads."""
    pool, meta = cache.pool, cache.metadata
    batch = key.shape[0]
    lib, stream = _native.library(), _native.stream_handle(pool.device)
    max_tokens = cache.max_pages_per_sequence * pool.page_size
    _native.check(lib.nq_nqkv_advance(
        slot_ids.data_ptr(), active_mask.data_ptr(), None, 1, batch, cache.max_sequences, pool.page_size, max_tokens,
        meta.sequence_lengths.data_ptr(), meta.page_counts.data_ptr(), meta.last_page_lens.data_ptr(),
        meta.hot_lengths.data_ptr(), stream))
    _native.check(lib.nq_nqkv_write(
        key.data_ptr(), value.data_ptr(), _native.dtype_tag(key.dtype), slot_ids.data_ptr(), active_mask.data_ptr(),
        None, 1, meta.sequence_lengths.data_ptr(), meta.page_indices.data_ptr(),
        pool.key_codes.data_ptr(), pool.key_betas.data_ptr(), pool.key_norms.data_ptr(),
        pool.value_codes.data_ptr(), pool.value_betas.data_ptr(), pool.value_norms.data_ptr(),
        pool.beta_table.data_ptr(), pool.beta_table.numel(), pool.value_beta_table.data_ptr(),
        pool.value_beta_table.numel(), cache.hot_keys.data_ptr(), cache.hot_values.data_ptr(),
        batch, 1, cache.max_sequences, cache.max_pages_per_sequence, pool.num_kv_heads, pool.head_dim, pool.page_size,
        0, None, None, *pool.hint_pointers(), stream))


def append_hot_k1_graph_safe(key: torch.Tensor, value: torch.Tensor, cache: NQKVHotColdCache, *,
                             slot_ids: torch.Tensor, active_mask: torch.Tensor) -> None:
    """Append one token per active row of one cache (nestquant/runtime/nqkv_graph_writer.py:263-289):
    key / value BF16 [batch, kv_heads, head_dim] land in the hot tail of slot_ids[r], and the
    device tables of the cache advance by one token.  An append that completes a page encodes
    and publishes that page into physical page page_indices[slot, ordinal] in the same launch, so
    the "hot page is full" state the reference refuses here never exists; what is refused instead
    is a sequence that already holds max_pages * page_size tokens, and a page ordinal that is not
    mapped to a physical page.  The checks read the tables on the host; the launch itself
    (`_launch_append_hot_k1_graph_safe`) does not and is capturable.

    A cache that shares its tables with other layers (BatchedNQKVCacheManager) must not be
    advanced once per layer: there `begin_step` + `write_layer` are the entry points."""
    _check_hot_k1_inputs(key, value, cache, slot_ids, active_mask)
    slots = slot_ids[active_mask].detach().cpu().tolist()
    if len(slots) != len(set(slots)):
        raise ValueError("active slot_ids must be unique")
    if any(not 0 <= slot < cache.max_sequences for slot in slots):
        raise ValueError("active slot_ids must be inside the cache")
    if slots:
        pool, meta = cache.pool, cache.metadata
        index = torch.tensor(slots, dtype=torch.long, device=pool.device)
        lengths = meta.sequence_lengths[index]
        if bool((lengths >= cache.max_pages_per_sequence * pool.page_size).any().item()):
            raise RuntimeError("sequence already fills its pages")
        completes = (lengths + 1) % pool.page_size == 0
        targets = meta.page_indices[index, lengths // pool.page_size]
        if bool((completes & ((targets < 0) | (targets >= pool.capacity))).any().item()):
            raise RuntimeError("the page this append completes is not mapped to a physical page")
    _launch_append_hot_k1_graph_safe(key, value, cache, slot_ids=slot_ids, active_mask=active_mask)


def launch_pack_full_hot_pages_graph_safe(cache: NQKVHotColdCache, *, boundary_mask: torch.Tensor,
                                          batched_encode: bool = False) -> None:
    """The page-boundary stage of the reference's decode graph
    (nestquant/runtime/nqkv_graph_pack.py:76-135): encode the full hot pages of the rows in
    `boundary_mask` and publish them.  Here the append that fills a page has already done both
    (`append_hot_k1_graph_safe`, `write_layer`), so after validating its arguments this launches
    nothing: the cache is in the state the reference reaches after this call."""
    del batched_encode
    if not isinstance(cache, NQKVHotColdCache):
        raise TypeError("cache must be an NQKVHotColdCache")
    if boundary_mask.dtype != torch.bool or tuple(boundary_mask.shape) != (cache.max_sequences,):
        raise ValueError("boundary_mask must be bool with cache capacity shape")
    if boundary_mask.device != cache.pool.device:
        raise ValueError("boundary_mask must be on the cache device")


# --------------------------------------------------------------------------------------
# multi-layer manager: step bookkeeping + the ragged writer
# --------------------------------------------------------------------------------------

class BatchedNQKVCacheManager:
    """Fixed-capacity, multi-layer NQKV cache.  All layers share one set of device tables
    (every layer holds the same number of tokens per slot) and every slot owns the fixed
    physical pages [slot * max_pages, (slot + 1) * max_pages) of each layer's pool."""

    def __init__(self, *, capacity: int, num_layers: int, num_kv_heads: int, head_dim: int,
                 max_cache_len: int, page_size: int, q: int, key_betas: Sequence[float],
                 value_betas: Sequence[float], dtype: torch.dtype, device: torch.device | str,
                 hints: bool = False) -> None:
        """`hints`: every layer's pool also keeps the decode hints (NQKVPagePool), four bits per block."""
        if dtype != torch.bfloat16:
            raise ValueError("the NQKV hot tails and writer are BF16")
        self.capacity, self.num_layers, self.page_size = capacity, num_layers, page_size
        self.max_pages = math.ceil(max_cache_len / page_size)
        self.max_tokens = self.max_pages * page_size
        target = torch.device(device)
        if target.type == "cuda" and target.index is None:
            target = torch.device("cuda", torch.cuda.current_device())
        self.device = target
        self.metadata = BatchedNQKVMetadata.create(capacity=capacity, max_pages_per_sequence=self.max_pages,
                                                   device=target)
        self.metadata.page_indices.copy_(
            torch.arange(capacity * self.max_pages, dtype=torch.int32, device=target).reshape(capacity, self.max_pages))
        self.layers = [
            NQKVHotColdCache(
                NQKVPagePool(capacity=capacity * self.max_pages, page_size=page_size, num_kv_heads=num_kv_heads,
                             head_dim=head_dim, q=q, key_betas=key_betas, value_betas=value_betas,
                             output_dtype=dtype, device=target, hints=hints),
                self.metadata, max_sequences=capacity, max_pages_per_sequence=self.max_pages)
            for _ in range(num_layers)
        ]
        self._sequence_of_slot: list[Hashable | None] = [None] * capacity
        # state of the step in flight (fixed-address tensors so graphs can be replayed)
        self.step_slot_ids = torch.arange(capacity, dtype=torch.int32, device=target)
        self.step_active = torch.zeros(capacity, dtype=torch.bool, device=target)
        self.step_counts = torch.zeros(capacity, dtype=torch.int32, device=target)
        self._step_rows = capacity
        self._step_uniform: int | None = 1
        # a prompt step's description on its way to the device: pinned host words, their device copy, and
        # the event that says the last copy has left the host words
        self._prompt_record: torch.Tensor | None = None
        self._prompt_stage: torch.Tensor | None = None
        self._prompt_stage_free: torch.cuda.Event | None = None

    # -- slots ---------------------------------------------------------------------------
    def register(self, sequence_id: Hashable, *, slot: int) -> None:
        self.register_batch([(sequence_id, slot)])

    def register_batch(self, assignments: Sequence[tuple[Hashable, int]], *, reset_tables: bool = True) -> None:
        """All-or-nothing: every assignment is checked before the first slot is taken.  With
        `reset_tables=False` the slots' device tables are left to the `begin_prompt_step` that must
        follow and name these slots as fresh."""
        assignments = list(assignments)
        slots = [slot for _, slot in assignments]
        names = [name for name, _ in assignments]
        if any(not 0 <= slot < self.capacity for slot in slots):
            raise ValueError("slot is outside cache capacity")
        if len(set(names)) != len(names) or any(name in self._sequence_of_slot for name in names):
            raise ValueError("sequence is already registered")      # nqkv_batch_manager.py:395-396
        if len(set(slots)) != len(slots) or any(self._sequence_of_slot[slot] is not None for slot in slots):
            raise RuntimeError("slot is already occupied")          # nqkv_batch_manager.py:398-399
        for name, slot in assignments:
            self._sequence_of_slot[slot] = name
        if reset_tables:
            self._reset_slot_tables(slots, active=True)

    def _reset_slot_tables(self, slots: Sequence[int], *, active: bool) -> None:
        """Zero lengths and counts of `slots` and set their activity flag: one fill per table and run
        of neighbouring slots (a batch admitted into slots 0..b-1 costs two launches, not 5 b)."""
        ordered = sorted(slots)
        meta = self.metadata
        start = 0
        while start < len(ordered):
            stop = start
            while stop + 1 < len(ordered) and ordered[stop + 1] == ordered[stop] + 1:
                stop += 1
            first, last = ordered[start], ordered[stop] + 1
            meta.active_mask[first:last] = active
            if meta.counters is not None:
                meta.counters[:, first:last] = 0
            else:
                for tensor in (meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths):
                    tensor[first:last] = 0
            start = stop + 1

    def release_slots(self, slots: Sequence[int]) -> tuple[Hashable, ...]:
        held = [slot for slot in dict.fromkeys(slots) if self._sequence_of_slot[slot] is not None]
        released = tuple(self._sequence_of_slot[slot] for slot in held)
        for slot in held:
            self._sequence_of_slot[slot] = None
        self._reset_slot_tables(held, active=False)
        return released

    def sequence_id(self, slot: int) -> Hashable | None:
        return self._sequence_of_slot[slot]

    def total_tokens(self, slot: int) -> int:
        """Host read of one slot's length (diagnostics and tests; never on the step path)."""
        return int(self.metadata.sequence_lengths[slot].item())

    # -- one step -------------------------------------------------------------------------
    def begin_step(self, *, rows: int, uniform_count: int | None) -> None:
        """Advance the device tables for a step over the first `rows` entries of
        step_slot_ids / step_active (and step_counts unless `uniform_count` is given).
        Graph-capturable: reads nothing on the host."""
        self._step_rows, self._step_uniform = rows, uniform_count
        meta = self.metadata
        _native.check(_native.library().nq_nqkv_advance(
            self.step_slot_ids.data_ptr(), self.step_active.data_ptr(),
            None if uniform_count is not None else self.step_counts.data_ptr(),
            0 if uniform_count is None else uniform_count, rows, self.capacity, self.page_size, self.max_tokens,
            meta.sequence_lengths.data_ptr(), meta.page_counts.data_ptr(), meta.last_page_lens.data_ptr(),
            meta.hot_lengths.data_ptr(), _native.stream_handle(self.device)))

    def begin_prompt_step(self, *, slot_ids: Sequence[int], counts: Sequence[int], fresh: Sequence[bool], width: int,
                          positions: torch.Tensor | None = None, last_token: torch.Tensor | None = None) -> None:
        """The head of a step that writes prompts, as one copy and one launch: row i writes its first
        counts[i] tokens into slot_ids[i]; `fresh[i]` restarts that slot's tables at zero and marks it
        active (a sequence registered with `reset_tables=False`).  Leaves step_slot_ids / step_counts /
        step_active as `set_batch_state` would, advances the tables as `begin_step` and fills, when
        given, positions [rows, width] (tokens held + column) and last_token [rows] (count - 1), both
        int64 on the device.  Host lists go to the device through pinned words, so nothing here waits."""
        rows = len(slot_ids)
        if not 1 <= rows <= self.capacity or len(counts) != rows or len(fresh) != rows:
            raise ValueError("slot_ids, counts and fresh must describe 1..capacity rows")
        for name, tensor, shape in (("positions", positions, (rows, width)), ("last_token", last_token, (rows,))):
            if tensor is not None and (tensor.dtype != torch.int64 or tuple(tensor.shape) != shape
                                       or not tensor.is_contiguous() or tensor.device != self.device):
                raise ValueError(f"{name} must be contiguous int64 {shape} on the cache's device")
        if self._prompt_record is None:
            self._prompt_record = torch.zeros(3 * self.capacity, dtype=torch.int32, device=self.device)
            self._prompt_stage = torch.zeros(3 * self.capacity, dtype=torch.int32, pin_memory=True)
            with torch.cuda.device(self.device):
                self._prompt_stage_free = torch.cuda.Event()
        else:
            self._prompt_stage_free.synchronize()             # the previous step's copy has read the words
        words = [int(s) for s in slot_ids] + [int(c) for c in counts] + [int(bool(f)) for f in fresh]
        self._prompt_stage[:3 * rows] = torch.tensor(words, dtype=torch.int32)
        self._prompt_record[:3 * rows].copy_(self._prompt_stage[:3 * rows], non_blocking=True)
        self._prompt_stage_free.record(torch.cuda.current_stream(self.device))
        self._step_rows, self._step_uniform = rows, None
        meta = self.metadata
        _native.check(_native.library().nq_prompt_step_begin(
            self._prompt_record.data_ptr(), rows, width, self.capacity, self.page_size, self.max_tokens,
            self.step_slot_ids.data_ptr(), self.step_counts.data_ptr(), self.step_active.data_ptr(),
            meta.sequence_lengths.data_ptr(), meta.page_counts.data_ptr(), meta.last_page_lens.data_ptr(),
            meta.hot_lengths.data_ptr(), meta.active_mask.data_ptr(),
            None if positions is None else positions.data_ptr(),
            None if last_token is None else last_token.data_ptr(), _native.stream_handle(self.device)))

    def begin_decode_step(self, *, rows: int, tokens: torch.Tensor, embedding: torch.Tensor,
                          positions: torch.Tensor, rotary: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """`begin_step(rows=rows, uniform_count=1)` and, in the same launch, the embedding rows of
        `tokens` (int64, `rows` entries; `embedding` BF16 [vocab, hidden]) and the rows of
        `positions` (int64, `rows` entries) of `rotary` (BF16 [2, positions, head_dim]: cos, sin).
        Returns (embedded [rows, hidden], rotary rows [2, rows, head_dim]).  Graph-capturable."""
        for name, tensor in (("tokens", tokens), ("positions", positions)):
            if tensor.dtype != torch.int64 or tensor.numel() != rows or not tensor.is_contiguous() or \
                    tensor.device != self.device:
                raise ValueError(f"{name} must be {rows} contiguous int64 entries on the cache's device")
        for name, tensor, ndim in (("embedding", embedding, 2), ("rotary", rotary, 3)):
            if tensor.dtype != torch.bfloat16 or tensor.ndim != ndim or not tensor.is_contiguous() or \
                    tensor.device != self.device or tensor.shape[-1] % 8:
                raise ValueError(f"{name} must be a contiguous BF16 table on the cache's device")
        if rotary.shape[0] != 2:
            raise ValueError("rotary holds the cos rows, then the sin rows: [2, positions, head_dim]")
        self._step_rows, self._step_uniform = rows, 1
        meta = self.metadata
        embedded = torch.empty((rows, embedding.shape[1]), dtype=torch.bfloat16, device=self.device)
        rotary_rows = torch.empty((2, rows, rotary.shape[2]), dtype=torch.bfloat16, device=self.device)
        _native.check(_native.library().nq_decode_step_begin(
            self.step_slot_ids.data_ptr(), self.step_active.data_ptr(), rows, self.capacity, self.page_size,
            self.max_tokens, meta.sequence_lengths.data_ptr(), meta.page_counts.data_ptr(),
            meta.last_page_lens.data_ptr(), meta.hot_lengths.data_ptr(), tokens.data_ptr(), embedding.data_ptr(),
            embedding.shape[0], embedding.shape[1], embedded.data_ptr(), positions.data_ptr(), rotary.data_ptr(),
            rotary.shape[1], rotary.shape[2], rotary_rows.data_ptr(), _native.stream_handle(self.device)))
        return embedded, rotary_rows

    def write_layer(self, layer_index: int, key: torch.Tensor, value: torch.Tensor, *,
                    rotate_keys: bool = False,
                    rope: tuple[torch.Tensor, torch.Tensor] | None = None) -> None:
        """Append this step's K/V rows [rows, tokens, kv_heads, head_dim] to one layer;
        `rotate_keys` Hadamard-rotates the new keys inside the kernel, `rope` (BF16 cos, sin
        [rows, tokens, head_dim]) applies the rotary embedding to them before that."""
        cache = self.layers[layer_index]
        pool, meta = cache.pool, self.metadata
        rows, tokens = key.shape[0], key.shape[1]
        if rows != self._step_rows:
            raise ValueError("key rows do not match the step in flight")
        uniform = self._step_uniform
        _native.check(_native.library().nq_nqkv_write(
            key.data_ptr(), value.data_ptr(), _native.dtype_tag(key.dtype), self.step_slot_ids.data_ptr(),
            self.step_active.data_ptr(), None if uniform is not None else self.step_counts.data_ptr(),
            0 if uniform is None else uniform, meta.sequence_lengths.data_ptr(), meta.page_indices.data_ptr(),
            pool.key_codes.data_ptr(), pool.key_betas.data_ptr(), pool.key_norms.data_ptr(),
            pool.value_codes.data_ptr(), pool.value_betas.data_ptr(), pool.value_norms.data_ptr(),
            pool.beta_table.data_ptr(), pool.beta_table.numel(), pool.value_beta_table.data_ptr(),
            pool.value_beta_table.numel(), cache.hot_keys.data_ptr(), cache.hot_values.data_ptr(),
            rows, tokens, self.capacity, self.max_pages, pool.num_kv_heads, pool.head_dim, self.page_size,
            int(rotate_keys), None if rope is None else rope[0].data_ptr(),
            None if rope is None else rope[1].data_ptr(), *pool.hint_pointers(), _native.stream_handle(self.device)))

    def append_and_attend(self, layer_index: int, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, *,
                          attention_scale: float, workspace: BatchedNQKVAttentionWorkspace, rotate: bool = False,
                          rope: tuple[torch.Tensor, torch.Tensor] | None = None, merge: bool = True
                          ) -> torch.Tensor | None:
        """One decode token per row: `write_layer` of this step's key/value rows [rows, kv_heads,
        head_dim] and `launch_nqkv_decode_attention` of the query [rows, query_heads, head_dim] over
        the layer in one launch (BF16; the same `rope` rows and `rotate` serve keys and queries).
        Graph-safe: no host reads, no allocation.  Returns workspace.output, or None when `merge`
        is false (the per-chunk results then wait in workspace.buffer for attention_output_stage)."""
        cache = self.layers[layer_index]
        pool, meta = cache.pool, self.metadata
        rows, heads, dim = query.shape
        if rows != self._step_rows or self._step_uniform != 1:
            raise ValueError("append_and_attend takes the rows of a decode step in flight, one token each")
        if not (query.dtype == key.dtype == value.dtype == torch.bfloat16):
            raise TypeError("append_and_attend takes BF16 queries, keys and values")
        if tuple(key.shape) != (rows, pool.num_kv_heads, dim) or key.shape != value.shape:
            raise ValueError("keys and values must have shape [rows, kv_heads, head_dim]")
        if not (query.is_contiguous() and key.is_contiguous() and value.is_contiguous()):
            raise ValueError("queries, keys and values must be contiguous")
        _native.check(_native.library().nq_nqkv_append_attention_decode(
            query.data_ptr(), key.data_ptr(), value.data_ptr(), meta.sequence_lengths.data_ptr(),
            pool.key_codes.data_ptr(), pool.key_betas.data_ptr(), pool.key_norms.data_ptr(),
            pool.value_codes.data_ptr(), pool.value_betas.data_ptr(), pool.value_norms.data_ptr(),
            pool.beta_table.data_ptr(), pool.beta_table.numel(), pool.value_beta_table.data_ptr(),
            pool.value_beta_table.numel(), meta.page_indices.data_ptr(), meta.page_counts.data_ptr(),
            meta.last_page_lens.data_ptr(), meta.hot_lengths.data_ptr(), meta.active_mask.data_ptr(),
            cache.hot_keys.data_ptr(), cache.hot_values.data_ptr(), self.step_slot_ids.data_ptr(),
            self.step_active.data_ptr(), rows, self.capacity, self.max_pages, heads, pool.num_kv_heads, dim,
            self.page_size, attention_scale, int(rotate), None if rope is None else rope[0].data_ptr(),
            None if rope is None else rope[1].data_ptr(), workspace.output.data_ptr() if merge else None,
            workspace.buffer.data_ptr(), workspace.buffer.numel(), *pool.hint_pointers(),
            _native.stream_handle(self.device)))
        return workspace.output if merge else None

    def resident_bytes(self) -> int:
        total = 0
        for cache in self.layers:
            total += cache.pool.resident_bytes
            total += 2 * cache.hot_keys.numel() * cache.hot_keys.element_size()
        return total
