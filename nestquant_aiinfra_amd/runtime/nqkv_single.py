"""The one-sequence surface of the NQKV4 cache, under the reference's names:

  PagedNQKVCache                              nestquant/runtime/paged_nqkv_cache.py:98-332
  NQKVAttentionWorkspace, nqkv_decode_attention_k1   nestquant/runtime/nqkv_attention_k1.py:600-760
  NQKVLlamaCache, install_nqkv_llama_backend  nestquant/runtime/nqkv_hf_backend.py:24-232

Nothing here has a kernel of its own: a sequence is one row of the batched operators
(`nqkv_decode_attention_batched_k1`, `nqkv_prefill_attention`, the ragged writer), and the
objects below keep the host-side ownership the reference's callers rely on (sequence ids, page
handles taken from a pool on demand, one independent page table per layer).  The batched cache
(`BatchedNQKVLlamaCache`) is the fast path; this one is for callers written against the
single-sequence names.
"""

from __future__ import annotations

import math
from collections.abc import Hashable, Sequence
from dataclasses import dataclass, field

import torch
from transformers.cache_utils import Cache
from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

from .nqkv import (BatchedNQKVAttentionWorkspace, BatchedNQKVMetadata, NQKVHotColdCache, NQKVPageHandle,
                   NQKVPagePool, PreparedNQKVPage, nqkv_decode_attention_batched_k1, nqkv_prefill_attention)
from .w4a4_linear import hadamard_cuda

NQKV_ATTENTION_NAME = "nestquant_nqkv_k1"
_SEQUENCE_ID = "batch0"


@dataclass
class _Sequence:
    slot: int
    pages: list[NQKVPageHandle] = field(default_factory=list)         # published, in table order
    reserved: list[NQKVPageHandle] = field(default_factory=list)      # taken from the pool, not yet in the table
    last_page_tokens: int = 0                                         # valid tokens of the newest published page


class PagedNQKVCache:
    """Logical sequences over a page pool: which sequence sits in which slot of the fixed-address
    page tables, and which physical pages it owns.  The tables are the BatchedNQKVMetadata tensors
    the kernels read; this class is their host-side owner for callers that allocate pages on demand
    (reserve, fill, publish) instead of giving every slot a fixed range of pages."""

    def __init__(self, pool: NQKVPagePool, *, max_sequences: int, max_pages_per_sequence: int) -> None:
        if not isinstance(pool, NQKVPagePool):
            raise TypeError("pool must be an NQKVPagePool")
        for name, value in (("max_sequences", max_sequences), ("max_pages_per_sequence", max_pages_per_sequence)):
            if isinstance(value, bool) or not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be a positive integer")
        self.pool, self.max_sequences, self.max_pages_per_sequence = pool, max_sequences, max_pages_per_sequence
        self.metadata = BatchedNQKVMetadata.create(capacity=max_sequences,
                                                   max_pages_per_sequence=max_pages_per_sequence, device=pool.device)
        meta = self.metadata
        # the reference's attribute names for the same tensors
        self.slot_ids, self.page_indptr, self.page_indices = meta.slot_ids, meta.page_indptr, meta.page_indices
        self.page_counts, self.last_page_len, self.hot_lengths = meta.page_counts, meta.last_page_lens, meta.hot_lengths
        self.sequence_lengths, self.active = meta.sequence_lengths, meta.active_mask
        self._by_id: dict[Hashable, _Sequence] = {}
        self._by_slot: list[Hashable | None] = [None] * max_sequences
        self._occupied = [False] * max_sequences

    # -- sequences -----------------------------------------------------------------------------
    @property
    def active_sequences(self) -> int:
        return len(self._by_id)

    def register(self, sequence_id: Hashable, *, slot: int | None = None) -> int:
        """Bind a sequence to a slot (the lowest free one when none is named) and clear its tables."""
        hash(sequence_id)
        if sequence_id in self._by_id:
            raise ValueError("sequence is already registered")
        if all(self._occupied):
            raise RuntimeError("NQKV sequence table is full")
        if slot is None:
            slot = self._occupied.index(False)
        else:
            if isinstance(slot, bool) or not isinstance(slot, int):
                raise TypeError("slot must be an integer or None")
            if not 0 <= slot < self.max_sequences:
                raise ValueError("slot is outside NQKV sequence capacity")
            if self._occupied[slot]:
                raise RuntimeError("requested NQKV slot is already active")
        self._occupied[slot] = True
        self._by_id[sequence_id] = _Sequence(slot)
        self._by_slot[slot] = sequence_id
        self._clear_tables(slot, active=True)
        return slot

    def release(self, sequence_id: Hashable) -> None:
        state = self._state(sequence_id)
        for handle in state.pages + state.reserved:
            self.pool.release(handle)
        self._clear_tables(state.slot, active=False)
        del self._by_id[sequence_id]
        self._by_slot[state.slot] = None
        self._occupied[state.slot] = False

    def _clear_tables(self, slot: int, *, active: bool) -> None:
        self.page_indices[slot].fill_(-1)
        for table in (self.page_counts, self.last_page_len, self.hot_lengths, self.sequence_lengths):
            table[slot] = 0
        self.active[slot] = active

    # -- pages ---------------------------------------------------------------------------------
    def reserve_page(self, sequence_id: Hashable) -> NQKVPageHandle:
        """Take a physical page for the sequence without showing it to the kernels yet."""
        state = self._state(sequence_id)
        if len(state.pages) + len(state.reserved) >= self.max_pages_per_sequence:
            raise RuntimeError("sequence exceeds max_pages_per_sequence")
        if state.pages and state.last_page_tokens != self.pool.page_size:
            raise RuntimeError("replace the partial last page before appending another page")
        handle = self.pool.allocate()
        state.reserved.append(handle)
        return handle

    def cancel_reserved_page(self, sequence_id: Hashable, handle: NQKVPageHandle) -> None:
        self._take_reservation(self._state(sequence_id), handle)
        self.pool.release(handle)

    def commit_prepared_page(self, sequence_id: Hashable, handle: NQKVPageHandle,
                             page: PreparedNQKVPage) -> NQKVPageHandle:
        """Copy a GPU-encoded page into a reserved physical page and publish it in the tables."""
        state = self._state(sequence_id)
        if handle not in state.reserved:
            raise RuntimeError("NQKV page handle is not reserved for this sequence")
        try:
            self.pool.store_prepared(handle, page)
        except Exception:
            self.cancel_reserved_page(sequence_id, handle)
            raise
        return self._publish(state, handle, page.valid_tokens)

    def append_prepared_page(self, sequence_id: Hashable, page: PreparedNQKVPage) -> NQKVPageHandle:
        return self.commit_prepared_page(sequence_id, self.reserve_page(sequence_id), page)

    def append_page(self, sequence_id: Hashable, page) -> NQKVPageHandle:
        """Append a host container (PackedNQKVPage)."""
        handle = self.reserve_page(sequence_id)
        try:
            self.pool.store(handle, page)
        except Exception:
            self.cancel_reserved_page(sequence_id, handle)
            raise
        return self._publish(self._state(sequence_id), handle, page.valid_tokens)

    def replace_last_page(self, sequence_id: Hashable, page) -> NQKVPageHandle:
        """Overwrite the newest page with a host container that holds at least as many tokens."""
        state = self._state(sequence_id)
        if not state.pages:
            raise RuntimeError("sequence has no page to replace")
        if page.valid_tokens < state.last_page_tokens:
            raise ValueError("replacement page cannot shrink the valid prefix")
        handle = state.pages[-1]
        self.pool.store(handle, page)
        state.last_page_tokens = page.valid_tokens
        self.last_page_len[state.slot] = page.valid_tokens
        self.sequence_lengths[state.slot] = self._cold_tokens(state)
        return handle

    def commit_graph_page(self, sequence_id: Hashable, handle: NQKVPageHandle) -> NQKVPageHandle:
        """Host ownership of a page that a kernel has already filled and counted in the tables."""
        state = self._state(sequence_id)
        self._take_reservation(state, handle, what="NQKV graph page handle is not reserved for this sequence")
        state.pages.append(handle)
        state.last_page_tokens = self.pool.page_size
        self.pool.mark_graph_stored(handle, valid_tokens=self.pool.page_size)
        return handle

    def _publish(self, state: _Sequence, handle: NQKVPageHandle, valid_tokens: int) -> NQKVPageHandle:
        self._take_reservation(state, handle)
        state.pages.append(handle)
        state.last_page_tokens = valid_tokens
        self.page_indices[state.slot, len(state.pages) - 1] = handle.page_id
        self.page_counts[state.slot] = len(state.pages)
        self.last_page_len[state.slot] = valid_tokens
        self.sequence_lengths[state.slot] = self._cold_tokens(state)
        return handle

    @staticmethod
    def _take_reservation(state: _Sequence, handle: NQKVPageHandle,
                          what: str = "NQKV page handle is not reserved for this sequence") -> None:
        if handle not in state.reserved:
            raise RuntimeError(what)
        state.reserved.remove(handle)

    # -- queries -------------------------------------------------------------------------------
    def slot(self, sequence_id: Hashable) -> int:
        return self._state(sequence_id).slot

    def handles(self, sequence_id: Hashable) -> tuple[NQKVPageHandle, ...]:
        return tuple(self._state(sequence_id).pages)

    def reserved_handles(self, sequence_id: Hashable) -> tuple[NQKVPageHandle, ...]:
        return tuple(self._state(sequence_id).reserved)

    def sequence_id(self, slot: int) -> Hashable:
        if isinstance(slot, bool) or not isinstance(slot, int):
            raise TypeError("slot must be an integer")
        if not 0 <= slot < self.max_sequences:
            raise ValueError("slot is outside NQKV sequence capacity")
        if not self._occupied[slot]:
            raise KeyError("NQKV slot is not active")
        return self._by_slot[slot]

    def total_tokens(self, sequence_id: Hashable) -> int:
        """Tokens in the sequence's packed pages (host bookkeeping: no device read)."""
        return self._cold_tokens(self._state(sequence_id))

    def _cold_tokens(self, state: _Sequence) -> int:
        return (len(state.pages) - 1) * self.pool.page_size + state.last_page_tokens if state.pages else 0

    def table_pointers(self) -> tuple[int, ...]:
        return self.metadata.pointers()

    def _state(self, sequence_id: Hashable) -> _Sequence:
        hash(sequence_id)
        try:
            return self._by_id[sequence_id]
        except KeyError as error:
            raise KeyError("sequence is not registered") from error


# --------------------------------------------------------------------------------------------
# attention of one sequence
# --------------------------------------------------------------------------------------------

class NQKVAttentionWorkspace(BatchedNQKVAttentionWorkspace):
    """Scratch and output of the one-sequence attention: the batched workspace with one row."""

    @classmethod
    def create(cls, cache: NQKVHotColdCache, *, query_heads: int, output_dtype: torch.dtype) -> "NQKVAttentionWorkspace":
        return super().create(cache, batch_size=1, query_heads=query_heads, output_dtype=output_dtype)


def nqkv_decode_attention_k1(query: torch.Tensor, cache: NQKVHotColdCache, sequence_id: Hashable, *,
                             scale: float | None = None, workspace: NQKVAttentionWorkspace | None = None) -> torch.Tensor:
    """Decode attention of one sequence over its packed pages and BF16 tail: query
    [query_heads, head_dim] (rotated like the stored keys) -> [query_heads, head_dim].  One row of
    nqkv_decode_attention_batched_k1, so there is no page-count limit."""
    if not isinstance(query, torch.Tensor) or query.ndim != 2:
        raise ValueError("query must have shape [query_heads, head_dim]")
    if not isinstance(cache, NQKVHotColdCache) or cache.cold_cache is cache:
        raise TypeError("cache must be an NQKVHotColdCache over a PagedNQKVCache")
    pool = cache.pool
    if query.device != pool.device or query.shape[1] != pool.head_dim:
        raise ValueError("query must match the cache CUDA device and head_dim")
    if query.shape[0] < 1 or query.shape[0] % pool.num_kv_heads:
        raise ValueError("query_heads must be a positive multiple of num_kv_heads")
    if cache.total_tokens(sequence_id) < 1:
        raise ValueError("cannot attend to an empty sequence")
    slot = cache.cold_cache.slot(sequence_id)
    if workspace is None:
        workspace = NQKVAttentionWorkspace.create(cache, query_heads=query.shape[0], output_dtype=query.dtype)
    out = nqkv_decode_attention_batched_k1(
        query.unsqueeze(0), cache, slot_ids=torch.tensor([slot], dtype=torch.int32, device=pool.device),
        active_mask=torch.ones(1, dtype=torch.bool, device=pool.device), scale=scale, workspace=workspace)
    return out[0]


# --------------------------------------------------------------------------------------------
# Hugging Face cache of one sequence
# --------------------------------------------------------------------------------------------

class NQKVLlamaCache(Cache):
    """One-sequence, multi-layer NQKV cache for a Llama decode loop driven by `model.forward`:
    every layer owns a pool, a page table and a tail, and `update` appends to the layer it is
    called for.  Prompts attend to the packed cache they have just been written to (the reference
    decodes the cache to BF16 and calls SDPA: the same values, nestquant/runtime/nqkv_hf_backend.py:146-171)
    and may arrive in several chunks.  Attention outputs follow the layout `LlamaAttention.forward`
    reshapes, [1, tokens, heads, head_dim]."""

    def __init__(self, *, num_layers: int, num_query_heads: int, num_kv_heads: int, head_dim: int,
                 max_cache_len: int, page_size: int, q: int, key_betas: Sequence[float],
                 value_betas: Sequence[float], dtype: torch.dtype, device: torch.device | str) -> None:
        super().__init__(layers=[])
        for name, value in (("num_layers", num_layers), ("num_query_heads", num_query_heads),
                            ("num_kv_heads", num_kv_heads), ("head_dim", head_dim),
                            ("max_cache_len", max_cache_len), ("page_size", page_size)):
            if isinstance(value, bool) or not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be a positive integer")
        if num_query_heads % num_kv_heads:
            raise ValueError("num_query_heads must be divisible by num_kv_heads")
        if dtype != torch.bfloat16:
            raise ValueError("the NQKV hot tails and writer are BF16")
        self.num_layers, self.num_query_heads, self.num_kv_heads = num_layers, num_query_heads, num_kv_heads
        self.head_dim, self._max_cache_len, self.page_size, self.dtype = head_dim, max_cache_len, page_size, dtype
        target = torch.device(device)
        if target.type == "cuda" and target.index is None:
            target = torch.device("cuda", torch.cuda.current_device())
        self.device = target
        pages = math.ceil(max_cache_len / page_size)
        self.layer_caches: list[NQKVHotColdCache] = []
        self.workspaces: list[NQKVAttentionWorkspace] = []
        for _ in range(num_layers):
            pool = NQKVPagePool(capacity=pages, page_size=page_size, num_kv_heads=num_kv_heads, head_dim=head_dim,
                                q=q, key_betas=key_betas, value_betas=value_betas, output_dtype=dtype, device=target)
            cache = NQKVHotColdCache(PagedNQKVCache(pool, max_sequences=1, max_pages_per_sequence=pages))
            cache.register(_SEQUENCE_ID)
            self.layer_caches.append(cache)
            self.workspaces.append(NQKVAttentionWorkspace.create(cache, query_heads=num_query_heads, output_dtype=dtype))
        self._slot = torch.zeros(1, dtype=torch.int32, device=target)
        self._active = torch.ones(1, dtype=torch.bool, device=target)

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int, *args, **kwargs):
        del args, kwargs
        self._validate_layer(layer_idx)
        if key_states.ndim != 4 or key_states.shape != value_states.shape:
            raise ValueError("NQKV cache update requires matching BHTD Key/Value")
        if key_states.shape[0] != 1:
            raise ValueError("NQKV Llama backend supports batch size one (BatchedNQKVLlamaCache takes more)")
        if key_states.shape[1] != self.num_kv_heads or key_states.shape[3] != self.head_dim:
            raise ValueError("Key/Value heads or head_dim disagree with NQKV cache")
        if key_states.device != self.device or key_states.dtype != self.dtype:
            raise ValueError("Key/Value must match NQKV cache device and dtype")
        rotated_key = hadamard_cuda(key_states.contiguous(), compute_dtype=torch.float32)
        self.layer_caches[layer_idx].append(_SEQUENCE_ID, rotated_key[0].transpose(0, 1).contiguous(),
                                            value_states[0].transpose(0, 1).contiguous())
        return rotated_key, value_states

    def attend(self, layer_idx: int, query_states: torch.Tensor, *, scale: float) -> torch.Tensor:
        self._validate_layer(layer_idx)
        if tuple(query_states.shape) != (1, self.num_query_heads, 1, self.head_dim):
            raise ValueError("NQKV K1 requires query shape [1, query_heads, 1, head_dim]")
        rotated = hadamard_cuda(query_states.contiguous(), compute_dtype=torch.float32)
        output = nqkv_decode_attention_k1(rotated[0, :, 0].contiguous(), self.layer_caches[layer_idx], _SEQUENCE_ID,
                                          scale=scale, workspace=self.workspaces[layer_idx])
        return output.view(1, 1, self.num_query_heads, self.head_dim)

    def prefill(self, layer_idx: int, query_states: torch.Tensor, *, scale: float) -> torch.Tensor:
        """Causal attention of the chunk `update` has just written, over the packed cache."""
        self._validate_layer(layer_idx)
        if (query_states.ndim != 4 or tuple(query_states.shape[:2]) != (1, self.num_query_heads)
                or query_states.shape[3] != self.head_dim):
            raise ValueError("NQKV prefill query has an incompatible BHTD shape")
        tokens = query_states.shape[2]
        cache = self.layer_caches[layer_idx]
        if cache.total_tokens(_SEQUENCE_ID) < tokens:
            raise ValueError("NQKV prefill attends to keys that update() has written first")
        rotated = hadamard_cuda(query_states.contiguous(), compute_dtype=torch.float32)
        return nqkv_prefill_attention(rotated.transpose(1, 2).contiguous(), cache, slot_ids=self._slot,
                                      active_mask=self._active, uniform_count=tokens, scale=scale)

    def get_seq_length(self, layer_idx: int = 0) -> int:
        self._validate_layer(layer_idx)
        return self.layer_caches[layer_idx].total_tokens(_SEQUENCE_ID)

    def get_max_length(self, layer_idx: int | None = None) -> int:
        if layer_idx is not None:
            self._validate_layer(layer_idx)
        return self._max_cache_len

    get_max_cache_shape = get_max_length

    @property
    def max_cache_len(self) -> int:          # a read-only property of the transformers Cache base class
        return self._max_cache_len

    def get_mask_sizes(self, query_length, layer_idx: int) -> tuple[int, int]:
        self._validate_layer(layer_idx)
        length = query_length if isinstance(query_length, int) else int(query_length.shape[0])
        return self.get_seq_length(layer_idx) + length, 0

    @property
    def batch_size(self) -> int:
        return 1

    @property
    def is_compileable(self) -> bool:
        return False

    def reorder_cache(self, beam_idx: torch.LongTensor) -> None:
        del beam_idx
        raise NotImplementedError("NQKV backend does not support beam search")

    def reset(self) -> None:
        for cache in self.layer_caches:
            cache.release(_SEQUENCE_ID)
            cache.register(_SEQUENCE_ID)

    def _validate_layer(self, layer_idx: int) -> None:
        if isinstance(layer_idx, bool) or not isinstance(layer_idx, int):
            raise TypeError("layer_idx must be an integer")
        if not 0 <= layer_idx < self.num_layers:
            raise ValueError("layer_idx is outside the NQKV layer range")


def _nqkv_attention_interface(module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                              attention_mask: torch.Tensor | None, **kwargs):
    del key, value, attention_mask          # the cache holds the keys; a prompt's mask is the causal one
    cache = getattr(module, "_nestquant_nqkv_cache", None)
    if not isinstance(cache, NQKVLlamaCache):
        raise RuntimeError("Llama attention module has no installed NQKV cache")
    if kwargs.get("dropout", 0.0) != 0.0:
        raise ValueError("NQKV backend supports inference dropout=0 only")
    scale = float(kwargs.get("scaling", module.scaling))
    if query.shape[2] == 1:
        return cache.attend(module.layer_idx, query, scale=scale), None
    return cache.prefill(module.layer_idx, query, scale=scale), None


def install_nqkv_llama_backend(model: torch.nn.Module, cache: NQKVLlamaCache) -> str:
    """Register the one-sequence attention and attach the cache to every Llama layer."""
    if not isinstance(model, torch.nn.Module):
        raise TypeError("model must be a torch module")
    if not isinstance(cache, NQKVLlamaCache):
        raise TypeError("cache must be an NQKVLlamaCache")
    ALL_ATTENTION_FUNCTIONS.register(NQKV_ATTENTION_NAME, _nqkv_attention_interface)
    attached = 0
    for module in model.modules():
        if module.__class__.__name__ == "LlamaAttention":
            if not 0 <= module.layer_idx < cache.num_layers:
                raise ValueError("Llama layer index disagrees with NQKV cache")
            module._nestquant_nqkv_cache = cache
            module.config._attn_implementation = NQKV_ATTENTION_NAME
            attached += 1
    if attached != cache.num_layers:
        raise ValueError(f"expected {cache.num_layers} LlamaAttention modules, found {attached}")
    if hasattr(model, "config"):
        model.config._attn_implementation = NQKV_ATTENTION_NAME
    return NQKV_ATTENTION_NAME
