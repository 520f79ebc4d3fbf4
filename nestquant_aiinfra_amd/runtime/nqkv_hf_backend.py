"""Hugging Face integration of the batched NQKV4 cache: a `transformers` Cache, the
AttentionInterface function, and a fixed-capacity runner with a captured decode step.

Mirrors BatchedNQKVLlamaCache / install_batched_nqkv_llama_backend
(nestquant/runtime/nqkv_batched_hf_backend.py:26-680) and BatchedNQKVLlamaRunner
(nestquant/runtime/nqkv_batched_runner.py:10-378).  What differs, and why:
  * one decode graph per batch width instead of a normal and a page-boundary graph, and no
    host read of hot lengths before a step: the writer kernel packs a page whenever one
    fills, from device-resident lengths;
  * post-RoPE key and query rotations run inside the writer and attention kernels;
  * the prefill attention output is returned as [batch, tokens, heads, dim], which is what
    `LlamaAttention.forward` reshapes (the reference returns the raw SDPA layout).
"""

from __future__ import annotations

from collections.abc import Hashable, Sequence

import torch
import torch.nn.functional as F
from transformers.cache_utils import Cache
from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

from .. import _native
from .nqkv import (BatchedNQKVAttentionWorkspace, BatchedNQKVCacheManager, launch_nqkv_decode_attention,
                   nqkv_prefill_attention)
from .w4a4_linear import hadamard_cuda

BATCHED_NQKV_ATTENTION_NAME = "nestquant_batched_nqkv_k1"


class BatchedNQKVLlamaCache(Cache):
    """Multi-layer fixed-capacity NQKV cache driven by scheduler slot state."""

    def __init__(self, *, capacity: int, num_layers: int, num_query_heads: int, num_kv_heads: int,
                 head_dim: int, max_cache_len: int, page_size: int, q: int, key_betas: Sequence[float],
                 value_betas: Sequence[float], dtype: torch.dtype, device: torch.device | str,
                 packed_prefill: bool = False, decode_hints: bool = False) -> None:
        """`packed_prefill` (an extension): prefill chunks attend to the packed cache instead of
        the BF16 keys and values of the chunk, so long prompts can be fed in pieces.  A chunk
        written into a slot that already holds tokens always takes that route.  `decode_hints` (an
        extension): the pools keep four more bits per block, with which the attention kernels skip the
        lattice searches of the KV decode (same outputs bit for bit)."""
        super().__init__(layers=[])
        for name, value in (("capacity", capacity), ("num_layers", num_layers),
                            ("num_query_heads", num_query_heads), ("num_kv_heads", num_kv_heads),
                            ("head_dim", head_dim), ("max_cache_len", max_cache_len), ("page_size", page_size)):
            if isinstance(value, bool) or not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be a positive integer")
        if num_query_heads % num_kv_heads:
            raise ValueError("num_query_heads must be divisible by num_kv_heads")
        self.manager = BatchedNQKVCacheManager(
            capacity=capacity, num_layers=num_layers, num_kv_heads=num_kv_heads, head_dim=head_dim,
            max_cache_len=max_cache_len, page_size=page_size, q=q, key_betas=key_betas,
            value_betas=value_betas, dtype=dtype, device=device, hints=decode_hints)
        self.capacity, self.num_layers = capacity, num_layers
        self.num_query_heads, self.num_kv_heads, self.head_dim = num_query_heads, num_kv_heads, head_dim
        self._max_cache_len = max_cache_len
        self.page_size, self.dtype, self.device = page_size, dtype, self.manager.device
        self.slot_ids = torch.arange(capacity, device=self.device, dtype=torch.int32)
        self.active_mask = torch.zeros(capacity, device=self.device, dtype=torch.bool)
        self.packed_prefill = bool(packed_prefill)
        self._continuation = False
        self._rows = capacity
        self._tokens: int | None = None
        self._workspaces: dict[int, BatchedNQKVAttentionWorkspace] = {}
        self._host_lengths = [0] * capacity      # host mirror of sequence lengths (admission checks)

    # -- slots ---------------------------------------------------------------------------
    def register(self, sequence_id: Hashable, *, slot: int) -> None:
        self.manager.register(sequence_id, slot=slot)
        self._host_lengths[slot] = 0

    def register_batch(self, assignments: Sequence[tuple[Hashable, int]], *, reset_tables: bool = True) -> None:
        assignments = list(assignments)
        self.manager.register_batch(assignments, reset_tables=reset_tables)
        for _, slot in assignments:
            self._host_lengths[slot] = 0

    def release_slots(self, slots: Sequence[int]) -> tuple[Hashable, ...]:
        for slot in slots:
            self._host_lengths[slot] = 0
        return self.manager.release_slots(slots)

    # -- step state ------------------------------------------------------------------------
    def set_batch_state(self, *, slot_ids: Sequence[int] | None = None, counts: Sequence[int] | None = None,
                        active_mask: torch.Tensor | None = None, write_mask: torch.Tensor | None = None,
                        width: int | None = None, fresh: Sequence[int] | None = None,
                        positions: torch.Tensor | None = None, last_token: torch.Tensor | None = None) -> None:
        """Eager (prefill) step.  Two forms:
          * slot_ids / counts: row i writes its first counts[i] tokens into slot_ids[i] (`width`, when
            given, bounds every count);
          * active_mask / write_mask, the reference's form (nestquant/runtime/nqkv_batched_hf_backend.py:147):
            bool [capacity] and bool [capacity, width]; row r is slot r and writes the prefix of
            `write_mask[r]` (masks that are not prefixes are rejected).
        Validates before anything changes, copies the row state to the fixed step tensors and advances
        the device tables.  With `fresh` (first form, `width` given: the slots among slot_ids whose
        sequences were registered with `reset_tables=False`) all of that is one copy and one launch
        (`BatchedNQKVCacheManager.begin_prompt_step`), which also fills `positions` and `last_token`."""
        if write_mask is not None or active_mask is not None:
            if slot_ids is not None or counts is not None:
                raise ValueError("give slot_ids / counts or active_mask / write_mask, not both")
            if (not isinstance(write_mask, torch.Tensor) or write_mask.dtype != torch.bool or write_mask.ndim != 2
                    or write_mask.shape[0] != self.capacity):
                raise ValueError("write_mask must be bool with shape [capacity, width]")
            if active_mask is None:
                active_mask = write_mask.any(dim=1)
            if active_mask.dtype != torch.bool or tuple(active_mask.shape) != (self.capacity,):
                raise ValueError("active_mask must be bool with shape [capacity]")
            host_mask = write_mask.detach().cpu()
            host_active = active_mask.detach().cpu().tolist()
            width = write_mask.shape[1]
            counts = [int(row.sum()) if live else 0 for row, live in zip(host_mask, host_active)]
            for row, count in zip(host_mask, counts):
                if count and not bool(row[:count].all()):
                    raise ValueError("write_mask rows must be prefixes: written tokens lead each row")
            slot_ids = list(range(self.capacity))
        if slot_ids is None or counts is None:
            raise ValueError("set_batch_state needs slot_ids and counts (or the two masks)")
        slot_ids, counts = [int(s) for s in slot_ids], [int(c) for c in counts]
        rows = len(slot_ids)
        if rows < 1 or rows > self.capacity or len(counts) != rows:
            raise ValueError("slot_ids and counts must describe 1..capacity rows")
        if len(set(slot_ids)) != rows:
            raise ValueError("a slot may appear once per step")
        for slot, count in zip(slot_ids, counts):
            if not 0 <= slot < self.capacity:
                raise ValueError("slot is outside cache capacity")
            if count < 0 or (width is not None and count > width):
                raise ValueError("a row writes between 0 and `width` tokens")
            if count and self.manager.sequence_id(slot) is None:
                raise RuntimeError("slot has no registered sequence")
            if self._host_lengths[slot] + count > self._max_cache_len:
                raise RuntimeError("sequence would exceed max_cache_len")
        self._continuation = any(self._host_lengths[slot] > 0 and count > 0 for slot, count in zip(slot_ids, counts))
        m = self.manager
        if fresh is not None:
            if width is None:
                raise ValueError("the one-launch form needs `width`")
            starting = set(int(slot) for slot in fresh)
            m.begin_prompt_step(slot_ids=slot_ids, counts=counts, fresh=[slot in starting for slot in slot_ids],
                                width=width, positions=positions, last_token=last_token)
        else:
            if positions is not None or last_token is not None:
                raise ValueError("positions / last_token are filled by the one-launch form (`fresh`) only")
            m.step_slot_ids[:rows].copy_(torch.tensor(slot_ids, dtype=torch.int32))
            m.step_counts[:rows].copy_(torch.tensor(counts, dtype=torch.int32))
            m.step_active[:rows].copy_(torch.tensor([c > 0 for c in counts]))
        for slot, count in zip(slot_ids, counts):
            self._host_lengths[slot] += count
        self._rows, self._tokens = rows, max(counts)
        if fresh is None:
            m.begin_step(rows=rows, uniform_count=None)

    def fail_closed(self, slots: Sequence[int]) -> None:
        """After a forward that raised: the step's table advance is not backed by keys and values in
        every layer, so the sequences it touched are dropped (tables zeroed, slots free), as the
        reference does on a failed prefill (nestquant/runtime/nqkv_batched_hf_backend.py:493-531)."""
        self.release_slots([slot for slot in slots if self.manager.sequence_id(slot) is not None])
        self._tokens = None

    def set_decode_execution_state(self, *, slot_ids: torch.Tensor, active_mask: torch.Tensor) -> None:
        """Decode rows for the steps that follow (device tensors of equal length <= capacity);
        copied into the fixed step tensors so that a captured graph sees new values."""
        rows = slot_ids.numel()
        if rows < 1 or rows > self.capacity or active_mask.numel() != rows:
            raise ValueError("decode state must describe 1..capacity rows")
        self.manager.step_slot_ids[:rows].copy_(slot_ids)
        self.manager.step_active[:rows].copy_(active_mask)
        self._rows, self._tokens = rows, 1

    def begin_decode_step(self) -> None:
        """Advance every active decode row by one token (graph-capturable)."""
        self.manager.begin_step(rows=self._rows, uniform_count=1)

    def note_decode_step(self, slots: Sequence[int]) -> None:
        """Host mirror of a (possibly graph-replayed) decode step."""
        for slot in slots:
            self._host_lengths[slot] += 1

    def require_room(self, slots: Sequence[int], tokens: int = 1) -> None:
        """Raises before a step that would take a slot past the cache length (the device tables
        clamp there, so the step itself would overwrite the newest tokens instead)."""
        for slot in slots:
            if self._host_lengths[slot] + tokens > self._max_cache_len:
                raise RuntimeError("sequence would exceed max_cache_len")

    # -- Cache protocol -------------------------------------------------------------------------
    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int, *args, **kwargs):
        del args, kwargs
        self._validate_layer(layer_idx)
        if self._tokens is None:
            raise RuntimeError("set_batch_state must run before model forward")
        if key_states.ndim != 4 or key_states.shape != value_states.shape:
            raise ValueError("batched NQKV update requires matching BHTD Key/Value")
        if tuple(key_states.shape) != (self._rows, self.num_kv_heads, key_states.shape[2], self.head_dim):
            raise ValueError("Key/Value shape disagrees with batched NQKV state")
        if key_states.device != self.device or key_states.dtype != self.dtype:
            raise ValueError("Key/Value must match the NQKV cache device and dtype")
        value_rows = value_states.transpose(1, 2).contiguous()
        if key_states.shape[2] == 1:
            # decode: rotation fused into the writer; attention reads the cache, not the return value
            self.manager.write_layer(layer_idx, key_states.transpose(1, 2).contiguous(), value_rows, rotate_keys=True)
            return key_states, value_states
        rotated_key = hadamard_cuda(key_states.contiguous(), compute_dtype=torch.float32)
        self.manager.write_layer(layer_idx, rotated_key.transpose(1, 2).contiguous(), value_rows)
        return rotated_key, value_states

    def _workspace(self, rows: int, dtype: torch.dtype) -> BatchedNQKVAttentionWorkspace:
        workspace = self._workspaces.get(rows)
        if workspace is None or workspace.output.dtype != dtype:
            workspace = BatchedNQKVAttentionWorkspace.create(
                self.manager.layers[0], batch_size=rows, query_heads=self.num_query_heads, output_dtype=dtype)
            self._workspaces[rows] = workspace
        return workspace

    def attend(self, layer_idx: int, query_states: torch.Tensor, *, scale: float) -> torch.Tensor:
        self._validate_layer(layer_idx)
        if tuple(query_states.shape) != (self._rows, self.num_query_heads, 1, self.head_dim):
            raise ValueError("batched NQKV decode requires [rows, heads, 1, dim]")
        query = query_states[:, :, 0].contiguous()
        m = self.manager
        output = launch_nqkv_decode_attention(
            query, m.layers[layer_idx], slot_ids=m.step_slot_ids, active_mask=m.step_active,
            attention_scale=scale, workspace=self._workspace(self._rows, query.dtype), rotate_query=True)
        return output.unsqueeze(1)                        # [rows, 1, heads, dim]

    def prefill(self, query_states: torch.Tensor, key_states: torch.Tensor, value_states: torch.Tensor,
                attention_mask: torch.Tensor | None, *, scale: float, layer_idx: int | None = None) -> torch.Tensor:
        """Prefill attends to the current BF16 K/V (keys already rotated by `update`), or, for a
        continuation chunk or with `packed_prefill`, causally to the packed cache that `update`
        has just extended."""
        rotated_query = hadamard_cuda(query_states.contiguous(), compute_dtype=torch.float32)
        if self.packed_prefill or self._continuation:
            if layer_idx is None:
                raise ValueError("attention over the packed cache needs the layer index")
            self._validate_layer(layer_idx)
            m = self.manager
            return nqkv_prefill_attention(
                rotated_query.transpose(1, 2).contiguous(), m.layers[layer_idx], slot_ids=m.step_slot_ids,
                active_mask=m.step_active, counts=m.step_counts, scale=scale)
        output = F.scaled_dot_product_attention(
            rotated_query, key_states, value_states, attn_mask=attention_mask, dropout_p=0.0,
            is_causal=attention_mask is None, scale=scale,
            enable_gqa=self.num_query_heads != self.num_kv_heads)
        return output.transpose(1, 2).contiguous()         # [rows, tokens, heads, dim]

    def get_seq_length(self, layer_idx: int = 0) -> int:
        self._validate_layer(layer_idx)
        return max(self._host_lengths, default=0)

    def get_max_length(self, layer_idx: int | None = None) -> int:
        if layer_idx is not None:
            self._validate_layer(layer_idx)
        return self._max_cache_len

    get_max_cache_shape = get_max_length

    @property
    def max_cache_len(self) -> int:
        return self._max_cache_len

    def get_mask_sizes(self, query_length, layer_idx: int) -> tuple[int, int]:
        self._validate_layer(layer_idx)
        length = query_length if isinstance(query_length, int) else int(query_length.shape[0])
        return self.get_seq_length(layer_idx) + length, 0

    @property
    def batch_size(self) -> int:
        return self.capacity

    @property
    def is_compileable(self) -> bool:
        return False

    def reorder_cache(self, beam_idx: torch.LongTensor) -> None:
        del beam_idx
        raise NotImplementedError("batched NQKV backend does not support beam search")

    def _validate_layer(self, layer_idx: int) -> None:
        if isinstance(layer_idx, bool) or not isinstance(layer_idx, int):
            raise TypeError("layer_idx must be an integer")
        if not 0 <= layer_idx < self.num_layers:
            raise ValueError("layer_idx is outside the batched NQKV layer range")


def _batched_nqkv_attention_interface(module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                      attention_mask: torch.Tensor | None, **kwargs):
    cache = getattr(module, "_nestquant_batched_nqkv_cache", None)
    if not isinstance(cache, BatchedNQKVLlamaCache):
        raise RuntimeError("Llama attention module has no batched NQKV cache")
    if kwargs.get("dropout", 0.0) != 0.0:
        raise ValueError("batched NQKV backend supports inference dropout=0 only")
    scale = float(kwargs.get("scaling", module.scaling))
    if query.shape[2] == 1:
        return cache.attend(module.layer_idx, query, scale=scale), None
    return cache.prefill(query, key, value, attention_mask, scale=scale, layer_idx=module.layer_idx), None


def install_batched_nqkv_llama_backend(model: torch.nn.Module, cache: BatchedNQKVLlamaCache) -> str:
    """Attach fixed-capacity batched NQKV attention to every Llama layer."""
    if not isinstance(model, torch.nn.Module):
        raise TypeError("model must be a torch module")
    if not isinstance(cache, BatchedNQKVLlamaCache):
        raise TypeError("cache must be a BatchedNQKVLlamaCache")
    ALL_ATTENTION_FUNCTIONS.register(BATCHED_NQKV_ATTENTION_NAME, _batched_nqkv_attention_interface)
    attached = 0
    for module in model.modules():
        if module.__class__.__name__ == "LlamaAttention":
            if not 0 <= module.layer_idx < cache.num_layers:
                raise ValueError("Llama layer index disagrees with batched NQKV cache")
            module._nestquant_batched_nqkv_cache = cache
            module.config._attn_implementation = BATCHED_NQKV_ATTENTION_NAME
            attached += 1
    if attached != cache.num_layers:
        raise ValueError(f"expected {cache.num_layers} LlamaAttention modules, found {attached}")
    if hasattr(model, "config"):
        model.config._attn_implementation = BATCHED_NQKV_ATTENTION_NAME
    return BATCHED_NQKV_ATTENTION_NAME


def greedy_sample_(logits: torch.Tensor, tokens: torch.Tensor, *, positions: torch.Tensor | None = None,
                   active_mask: torch.Tensor | None = None, history: torch.Tensor | None = None,
                   cursors: torch.Tensor | None = None, workspace: torch.Tensor | None = None) -> torch.Tensor:
    """Device-side GreedyHostSampler (nestquant/runtime/inference_engine.py:63-69): writes the
    argmax of logits [rows, vocab] (ties: lowest index) into tokens (int64, `rows` entries), in
    place, for the rows of `active_mask` (bool [rows]; all when None); advances `positions`
    (int64, `rows` entries) by one and appends to `history` (int64 [steps, rows]) at
    `cursors` (int32 [rows]), which it advances.  One launch; graph-safe when `workspace`
    (`greedy_sample_workspace(rows, device)`, reusable by calls that do not overlap) is given."""
    if logits.ndim != 2 or logits.stride(1) != 1:
        raise ValueError("sampler logits must have shape [requests, vocabulary] with contiguous rows")
    rows, vocab = logits.shape
    device = logits.device
    if device.type != "cuda":
        raise ValueError("tensors must live on the GPU (device type 'cuda' under ROCm)")
    for name, tensor, dtype in (("tokens", tokens, torch.int64), ("positions", positions, torch.int64),
                                ("history", history, torch.int64), ("cursors", cursors, torch.int32),
                                ("active_mask", active_mask, torch.bool)):
        if tensor is None:
            continue
        if tensor.dtype != dtype or tensor.device != device or not tensor.is_contiguous():
            raise ValueError(f"{name} must be a contiguous {dtype} tensor on the logits' device")
    if tokens.numel() != rows or (positions is not None and positions.numel() != rows) or (
            active_mask is not None and active_mask.numel() != rows):
        raise ValueError("tokens, positions and active_mask hold one entry per row of logits")
    steps = 0
    if history is not None:
        if cursors is None or cursors.numel() != rows or history.ndim != 2 or history.shape[1] != rows:
            raise ValueError("history must be [steps, rows] with one cursor per row")
        steps = history.shape[0]

    if workspace is None:
        workspace = greedy_sample_workspace(rows, device)
    elif workspace.dtype != torch.uint8 or workspace.device != device or not workspace.is_contiguous():
        raise ValueError("workspace must come from greedy_sample_workspace on the logits' device")

    def ptr(tensor):
        return None if tensor is None else tensor.data_ptr()

    _native.check(_native.library().nq_greedy_sample(
        logits.data_ptr(), _native.dtype_tag(logits.dtype), rows, vocab, logits.stride(0), ptr(active_mask),
        tokens.data_ptr(), ptr(positions), ptr(history), steps, ptr(cursors), workspace.data_ptr(),
        workspace.numel(), _native.stream_handle(device)))
    return tokens


def greedy_sample_workspace(rows: int, device: torch.device) -> torch.Tensor:
    """Zeroed scratch of greedy_sample_ for up to `rows` rows."""
    return torch.zeros(_native.library().nq_greedy_sample_workspace_bytes(rows), dtype=torch.uint8, device=device)


class BatchedNQKVLlamaRunner:
    """Fixed-capacity prefill / decode driver over a causal Llama model and an NQKV cache.

    Decode steps of width w in {1, 2, 4, ..., capacity} are captured once as HIP graphs
    (`capture`); active rows are compacted to the smallest width that holds them.  A step
    reads nothing from the device: token ids, positions, slot ids and masks are copied into
    the graph's fixed input tensors, the graph is replayed, logits are returned.  The captured
    step ends with the greedy sampler writing each active row's next token and position back
    into those input tensors, so `decode_greedy` replays it many times between host reads.
    """

    GREEDY_HISTORY_STEPS = 256
    takes_slot_lists = True          # the engine may call prefill_slots / decode with slots= instead of masks

    def __init__(self, model: torch.nn.Module, cache: BatchedNQKVLlamaCache, *,
                 fused_decode: bool | None = None, fused_prefill: bool | None = None,
                 expand_weights: bool = False, stage_linear_pairs=None) -> None:
        """`fused_decode` / `fused_prefill`: run decode steps through FusedLlamaDecodeStep and prompts
        through FusedLlamaPrefillStep instead of the module graph; None = whenever the model
        qualifies.  `expand_weights`: the fused decode step keeps and streams BF16 copies of the
        projection weights; `stage_linear_pairs`: which input stages share a launch with their
        linears (see FusedLlamaDecodeStep; None = all, () = none)."""
        if not isinstance(model, torch.nn.Module):
            raise TypeError("model must be a torch module")
        if not isinstance(cache, BatchedNQKVLlamaCache):
            raise TypeError("cache must be a BatchedNQKVLlamaCache")
        if model.training:
            raise ValueError("model must be in eval mode")
        device = next(model.parameters()).device
        if device.type != "cuda" or device != cache.device:
            raise ValueError("model and NQKV cache must share one CUDA device")
        self.model, self.cache, self.device = model, cache, device
        self.batch_size, self.max_cache_len = cache.capacity, cache.max_cache_len
        self._generation = [0] * self.batch_size
        self._graphs: dict[int, tuple[torch.cuda.CUDAGraph, torch.Tensor, torch.Tensor, torch.Tensor]] = {}
        # (rows, width) -> captured fused prefill with last-token logits: graph, tokens, positions, keep, logits
        self._prefill_graphs: dict[tuple[int, int], tuple] = {}
        self.prefill_graph_replay_counts: dict[tuple[int, int], int] = {}
        self._greedy: dict[int, tuple[torch.Tensor, ...]] = {}       # width -> (history, cursors, sampler scratch)
        self.graph_replay_counts: dict[int, int] = {}
        self._decode_state: tuple | None = None      # (width, slots) the step tensors were last set for
        self.fused_step = None
        if fused_decode is None or fused_decode:
            from .llama_decode_step import FusedLlamaDecodeStep, UnsupportedForFusedDecode
            try:
                self.fused_step = FusedLlamaDecodeStep(model, cache, expand_weights=expand_weights,
                                                       stage_linear_pairs=stage_linear_pairs)
            except UnsupportedForFusedDecode:
                if fused_decode:
                    raise
        self.fused_prefill = None
        if fused_prefill is None or fused_prefill:
            from .llama_decode_step import FusedLlamaPrefillStep, UnsupportedForFusedDecode
            try:
                self.fused_prefill = FusedLlamaPrefillStep(model, cache)
            except UnsupportedForFusedDecode:
                if fused_prefill:
                    raise

    @property
    def graph_captured(self) -> bool:
        return bool(self._graphs)

    # -- prefill -------------------------------------------------------------------------------
    def _check_reference_rows(self, input_ids: torch.Tensor, positions: torch.Tensor, mask: torch.Tensor,
                              valid_lengths: torch.Tensor) -> None:
        """Argument checks of the reference's runner (nestquant/runtime/nqkv_batched_runner.py:72-100)."""
        if input_ids.dtype != torch.long or input_ids.ndim != 2:
            raise ValueError("input_ids must be rank-2 torch.long")
        if input_ids.shape[0] != self.batch_size:
            raise ValueError("input batch must equal fixed runner capacity")
        if positions.dtype != torch.long or positions.shape != input_ids.shape:
            raise ValueError("positions must be torch.long and match input_ids")
        if mask.dtype != torch.bool or mask.shape != input_ids.shape:
            raise ValueError("write_mask must be bool and match input_ids")
        if valid_lengths.dtype != torch.long or tuple(valid_lengths.shape) != (self.batch_size,):
            raise ValueError("valid_lengths must have shape [batch_size]")
        if any(tensor.device != self.device for tensor in (input_ids, positions, mask, valid_lengths)):
            raise ValueError("runner inputs must be on the model CUDA device")
        if bool(mask.any().item()):
            written = positions[mask]
            if int(written.min().item()) < 0:
                raise ValueError("written positions must be non-negative")
            if int(written.max().item()) >= self.max_cache_len:
                raise ValueError("written positions exceed the NQKV cache")

    @torch.inference_mode()
    def prefill(self, input_ids: torch.Tensor) -> torch.Tensor:
        """Every fixed row takes its whole row of input_ids [capacity, width] as a fresh prompt (the
        warm-up call of the reference's engine, nestquant/runtime/nqkv_batched_runner.py:171-187)."""
        if input_ids.dtype != torch.long or input_ids.ndim != 2:
            raise ValueError("input_ids must be rank-2 torch.long")
        if input_ids.shape[0] != self.batch_size or input_ids.device != self.device:
            raise ValueError("input_ids batch or device does not match the runner")
        width = input_ids.shape[1]
        if width < 1 or width > self.max_cache_len:
            raise ValueError("prefill width is outside the NQKV cache")
        return self.prefill_slots(input_ids, slots=list(range(self.batch_size)), lengths=[width] * self.batch_size)

    @torch.inference_mode()
    def prefill_slots(self, input_ids: torch.Tensor, *, slots: Sequence[int] | None = None,
                      lengths: Sequence[int] | None = None, positions: torch.Tensor | None = None,
                      last_token_logits: bool = False, write_mask: torch.Tensor | None = None,
                      valid_lengths: torch.Tensor | None = None) -> torch.Tensor:
        """Prefill `slots[i]` with the first `lengths[i]` tokens of row i of input_ids
        [rows, width] (right padded).  New slots are registered.  Returns logits [rows, width, vocab],
        or, with `last_token_logits`, only those of every row's last token, [rows, 1, vocab]
        (what sampling the first new token needs: the LM head then runs on `rows` vectors).

        The reference's form (RaggedDecodeBackend, nestquant/runtime/inference_engine.py:14-32) is
        taken too: input_ids / positions / write_mask [capacity, width] and valid_lengths [capacity],
        row r being slot r and writing the prefix `write_mask[r]` marks; logits then come back as
        [capacity, width, vocab] with zero rows for slots that wrote nothing.

        A forward that raises leaves no slot half written: the sequences of the rows that were
        writing are dropped and their slots freed before the exception travels on."""
        if write_mask is not None:
            if slots is not None or lengths is not None:
                raise ValueError("give slots / lengths or write_mask / valid_lengths, not both")
            if positions is None or valid_lengths is None:
                raise ValueError("the masked form needs positions and valid_lengths")
            self._check_reference_rows(input_ids, positions, write_mask, valid_lengths)
            host_mask = write_mask.detach().cpu()
            counts = [int(row.sum()) for row in host_mask]
            for row, count in zip(host_mask, counts):
                if count and not bool(row[:count].all()):
                    raise ValueError("write_mask rows must be prefixes: written tokens lead each row")
            live = [slot for slot, count in enumerate(counts) if count]
            held = valid_lengths.detach().cpu().tolist()
            for slot in live:
                if held[slot] != self.cache._host_lengths[slot] + counts[slot]:
                    raise ValueError("valid_lengths of a writing row must equal the tokens it held plus those it writes")
            full = None
            if live:
                index = torch.tensor(live, dtype=torch.long, device=self.device)
                part = self.prefill_slots(input_ids[index], slots=live, lengths=[counts[s] for s in live],
                                          positions=positions[index], last_token_logits=last_token_logits)
                full = torch.zeros((self.batch_size, *part.shape[1:]), dtype=part.dtype, device=self.device)
                full[index] = part
            else:
                vocab = self.model.config.vocab_size
                full = torch.zeros((self.batch_size, 1 if last_token_logits else input_ids.shape[1], vocab),
                                   dtype=next(self.model.parameters()).dtype, device=self.device)
            return full
        if slots is None or lengths is None:
            raise ValueError("prefill_slots needs slots and lengths (or write_mask and valid_lengths)")
        rows, width = input_ids.shape
        slots, lengths = [int(s) for s in slots], [int(n) for n in lengths]
        if len(slots) != rows or len(lengths) != rows:
            raise ValueError("slots and lengths must have one entry per row")
        if len(set(slots)) != rows or any(not 0 <= slot < self.batch_size for slot in slots):
            raise ValueError("slots must be distinct and inside the runner's capacity")
        if any(not 0 <= length <= width for length in lengths):
            raise ValueError("a row holds between 0 and `width` prompt tokens")
        if last_token_logits and not all(1 <= length <= width for length in lengths):
            raise ValueError("last_token_logits needs at least one token in every row")
        for slot, length in zip(slots, lengths):
            if self.cache._host_lengths[slot] + length > self.max_cache_len:
                raise RuntimeError("sequence would exceed max_cache_len")
        one_launch = positions is None          # the step's head as one copy and one launch, positions included
        if positions is not None:
            if positions.dtype != torch.long or tuple(positions.shape) != (rows, width) or positions.device != self.device:
                raise ValueError("positions must be torch.long [rows, width] on the model device")
            written = torch.arange(width, device=self.device)[None, :] < torch.tensor(lengths, device=self.device)[:, None]
            if bool(written.any().item()):
                inside = positions[written]
                if int(inside.min().item()) < 0 or int(inside.max().item()) >= self.max_cache_len:
                    raise ValueError("written positions must lie in [0, max_cache_len)")
                # tokens are appended at the cache's own length while RoPE turns them by `positions`: the
                # two must name the same place, or keys would be stored at one position and rotated for another
                starts = torch.tensor([self.cache._host_lengths[s] for s in slots], device=self.device)
                expected = starts[:, None] + torch.arange(width, device=self.device)[None, :]
                if bool(((positions != expected) & written).any().item()):
                    raise ValueError("written positions must continue each slot's sequence: tokens already held + column")
        fresh = [slot for slot in slots if self.cache.manager.sequence_id(slot) is None]
        for slot in fresh:
            self._generation[slot] += 1
        self.cache.register_batch([(f"slot-{slot}-generation-{self._generation[slot]}", slot) for slot in fresh],
                                  reset_tables=not one_launch)
        self._decode_state = None
        continuation = any(self.cache._host_lengths[slot] > 0 and length > 0 for slot, length in zip(slots, lengths))
        captured = None
        if last_token_logits and not continuation and not self.cache.packed_prefill:
            captured = self._prefill_graphs.get((rows, width))
        keep = None
        if one_launch:
            if captured is not None:
                positions, keep = captured[2], captured[3]           # the graph's own inputs, filled in place
            else:
                positions = torch.empty((rows, width), dtype=torch.long, device=self.device)
                keep = torch.empty(rows, dtype=torch.long, device=self.device) if last_token_logits else None
            try:
                self.cache.set_batch_state(slot_ids=slots, counts=lengths, width=width, fresh=fresh,
                                           positions=positions, last_token=keep)
            except Exception:
                self.cache.release_slots(fresh)                      # registered above, tables never reset
                raise
        else:
            self.cache.set_batch_state(slot_ids=slots, counts=lengths, width=width)
            if last_token_logits:
                keep = torch.tensor([length - 1 for length in lengths], dtype=torch.long, device=self.device)
        try:
            if captured is not None:
                graph, graph_ids, graph_positions, graph_keep, logits = captured
                graph_ids.copy_(input_ids)
                if not one_launch:
                    graph_positions.copy_(positions)
                    graph_keep.copy_(keep)
                graph.replay()
                self.prefill_graph_replay_counts[(rows, width)] += 1
                return logits.clone()
            if self.fused_prefill is not None:
                return self.fused_prefill(input_ids, positions, keep=keep)
            output = self.model(input_ids=input_ids, position_ids=positions, past_key_values=self.cache, use_cache=True)
        except Exception:
            self.cache.fail_closed([slot for slot, length in zip(slots, lengths) if length])
            raise
        if keep is not None:
            return output.logits[torch.arange(rows, device=self.device), keep].unsqueeze(1)
        return output.logits

    @torch.inference_mode()
    def capture_prefill(self, *, rows: int, width: int) -> None:
        """Capture the fused prefill of `rows` fresh prompts of up to `width` tokens (the form with the last
        token's logits only, which is what an engine asks for) as one HIP graph.  A prompt of 128 tokens is
        bound by the host issuing its 270 launches; replayed from a graph it is bound by its kernels.
        `prefill_slots(..., last_token_logits=True)` then replays the graph whenever it is called with
        exactly [rows, width] tokens for slots that hold nothing yet; the row lengths may be anything up
        to `width` (they are read on the device).  Captured on rows that write nothing, so the cache is
        left as it was; same logits and cache contents as the un-captured call, bit for bit."""
        if self.fused_prefill is None:
            raise RuntimeError("capture_prefill needs the fused prefill step (fused_prefill=None or True on a model that qualifies)")
        if not 1 <= rows <= self.batch_size or not 1 <= width <= self.max_cache_len:
            raise ValueError("rows must be in [1, capacity] and width in [1, max_cache_len]")
        if self.cache.packed_prefill:
            raise RuntimeError("a cache with packed_prefill attends over the cache in every prefill: nothing to capture")
        cache, manager = self.cache, self.cache.manager
        meta = manager.metadata
        saved = [t.clone() for t in (meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths)]
        ids = torch.zeros((rows, width), dtype=torch.long, device=self.device)
        positions = torch.arange(width, device=self.device).repeat(rows, 1)
        keep = torch.zeros(rows, dtype=torch.long, device=self.device)
        manager.step_slot_ids[:rows].copy_(torch.arange(rows, dtype=torch.int32))
        manager.step_counts[:rows].zero_()
        manager.step_active[:rows].zero_()                   # inactive rows: the writer stores nothing
        cache._rows, cache._tokens, cache._continuation = rows, width, False
        self._decode_state = None
        stream = torch.cuda.Stream(device=self.device)
        stream.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(stream):
            for _ in range(2):
                manager.begin_step(rows=rows, uniform_count=None)
                self.fused_prefill(ids, positions, keep=keep)
            stream.synchronize()
            manager.begin_step(rows=rows, uniform_count=None)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                logits = self.fused_prefill(ids, positions, keep=keep)
        torch.cuda.current_stream(self.device).wait_stream(stream)
        for tensor, value in zip((meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths), saved):
            tensor.copy_(value)
        cache._tokens = None
        self._prefill_graphs[(rows, width)] = (graph, ids, positions, keep, logits)
        self.prefill_graph_replay_counts[(rows, width)] = 0

    def release_slots(self, slots: Sequence[int]) -> None:
        self.cache.release_slots(slots)

    def clear_slots(self, slot_mask: torch.Tensor) -> None:
        """Release the slots marked in a bool mask [capacity] (the reference's name for release)."""
        if slot_mask.dtype != torch.bool or tuple(slot_mask.shape) != (self.batch_size,):
            raise ValueError("slot_mask must be bool with shape [batch_size]")
        if slot_mask.device != self.device:
            raise ValueError("slot_mask must be on the model device")
        self.release_slots(slot_mask.nonzero(as_tuple=False).flatten().cpu().tolist())

    # -- decode --------------------------------------------------------------------------------
    def _check_pairs(self) -> None:
        """A one-launch (input stage + linear) pair whose consumers gave up waiting for the encoder has
        left outputs unwritten in some earlier step.  The step goes back to two launches per pair for
        good, the captured graphs (which hold the one-launch form) are dropped, and the caller is told."""
        step = self.fused_step
        if step is not None and step.pairs_failed():
            torch.cuda.synchronize(self.device)
            step.disable_pairs()
            self._graphs.clear()
            self._greedy.clear()
            self._decode_state = None
            raise RuntimeError("a fused input stage + linear launch gave up waiting for its encoder: results since the "
                               "last check are invalid; decode steps now use two launches per pair (capture again)")

    def _step(self, tokens: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        if self.fused_step is not None:
            return self.fused_step(tokens, positions, advance=True)
        self.cache.begin_decode_step()
        return self.model(input_ids=tokens, position_ids=positions, past_key_values=self.cache,
                          use_cache=True).logits

    @torch.inference_mode()
    def decode_eager(self, tokens: torch.Tensor, *, slots: Sequence[int], positions: torch.Tensor) -> torch.Tensor:
        """One un-captured decode step for `slots` (tokens, positions: [rows, 1])."""
        rows = len(slots)
        self._check_pairs()
        self.cache.require_room(slots)
        self._decode_state = None
        self.cache.set_decode_execution_state(
            slot_ids=torch.tensor(list(slots), dtype=torch.int32, device=self.device),
            active_mask=torch.ones(rows, dtype=torch.bool, device=self.device))
        logits = self._step(tokens, positions)
        self.cache.note_decode_step(slots)
        return logits

    @torch.inference_mode()
    def capture(self, sample_token: torch.Tensor | Sequence[int] | None = None, *, positions: torch.Tensor | None = None,
                active_mask: torch.Tensor | None = None, valid_lengths: torch.Tensor | None = None,
                widths: Sequence[int] | None = None) -> None:
        """Capture one decode graph per batch width.  The tables are restored afterwards, so capture
        leaves the cache unchanged.  The reference's arguments (sample_token, positions, active_mask,
        valid_lengths: nestquant/runtime/nqkv_batched_runner.py:227-299) are accepted and not needed:
        the graphs are captured on inactive rows and read their inputs from fixed tensors."""
        del positions, active_mask, valid_lengths
        if widths is None and sample_token is not None and not isinstance(sample_token, torch.Tensor):
            widths = list(sample_token)
        if widths is None:
            widths, width = [], 1
            while width < self.batch_size:
                widths.append(width)
                width *= 2
            widths.append(self.batch_size)
        self._decode_state = None
        meta = self.cache.manager.metadata
        saved = [t.clone() for t in (meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths)]
        stream = torch.cuda.Stream(device=self.device)
        for width in widths:
            tokens = torch.zeros((width, 1), dtype=torch.long, device=self.device)
            positions = torch.zeros((width, 1), dtype=torch.long, device=self.device)
            self.cache.set_decode_execution_state(
                slot_ids=torch.arange(width, dtype=torch.int32, device=self.device),
                active_mask=torch.zeros(width, dtype=torch.bool, device=self.device))   # inactive: writes nothing
            stream.wait_stream(torch.cuda.current_stream(self.device))
            with torch.cuda.stream(stream):
                for _ in range(2):
                    self._step(tokens, positions)
                stream.synchronize()
                history = torch.zeros((self.GREEDY_HISTORY_STEPS, width), dtype=torch.long, device=self.device)
                cursors = torch.zeros(width, dtype=torch.int32, device=self.device)
                scratch = greedy_sample_workspace(width, self.device)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=stream):
                    logits = self._step(tokens, positions)
                    greedy_sample_(logits.view(width, -1), tokens, positions=positions,
                                   active_mask=self.cache.manager.step_active[:width], history=history,
                                   cursors=cursors, workspace=scratch)
            torch.cuda.current_stream(self.device).wait_stream(stream)
            self._graphs[width] = (graph, tokens, positions, logits)
            self._greedy[width] = (history, cursors, scratch)
            self.graph_replay_counts[width] = 0
        for tensor, value in zip((meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths), saved):
            tensor.copy_(value)

    @torch.inference_mode()
    def decode(self, tokens: torch.Tensor, *, slots: Sequence[int] | None = None, positions: torch.Tensor,
               active_mask: torch.Tensor | None = None, valid_lengths: torch.Tensor | None = None) -> torch.Tensor:
        """One captured decode step: tokens / positions [rows, 1] for `slots`; logits [rows, 1, vocab].
        The reference's form (tokens / positions / active_mask [capacity, 1], valid_lengths [capacity];
        row r is slot r) returns [capacity, 1, vocab] with zero rows for inactive slots."""
        if active_mask is not None:
            if slots is not None:
                raise ValueError("give slots or active_mask, not both")
            if valid_lengths is None:
                raise ValueError("the masked form needs valid_lengths")
            self._check_reference_rows(tokens, positions, active_mask, valid_lengths)
            live = active_mask[:, 0].nonzero(as_tuple=False).flatten().cpu().tolist()
            vocab = self.model.config.vocab_size
            if not live:
                return torch.zeros((*tokens.shape, vocab), dtype=next(self.model.parameters()).dtype, device=self.device)
            index = torch.tensor(live, dtype=torch.long, device=self.device)
            part = self.decode(tokens[index], slots=live, positions=positions[index])
            full = torch.zeros((self.batch_size, *part.shape[1:]), dtype=part.dtype, device=self.device)
            full[index] = part
            return full
        if slots is None:
            raise ValueError("decode needs slots (or active_mask and valid_lengths)")
        self._check_pairs()
        rows = len(slots)
        width = next((w for w in sorted(self._graphs) if w >= rows), None)
        if width is None:
            return self.decode_eager(tokens, slots=slots, positions=positions)
        self.cache.require_room(slots)
        graph, graph_tokens, graph_positions, logits = self._graphs[width]
        graph_tokens[:rows].copy_(tokens)
        graph_positions[:rows].copy_(positions)
        state = (width, tuple(slots))
        if state != self._decode_state:
            # the step tensors still hold this row layout when consecutive steps decode the same slots
            padded_slots = list(slots) + [0] * (width - rows)
            self.cache.set_decode_execution_state(
                slot_ids=torch.tensor(padded_slots, dtype=torch.int32, device=self.device),
                active_mask=torch.tensor([True] * rows + [False] * (width - rows), device=self.device))
            self._decode_state = state
        graph.replay()
        self.graph_replay_counts[width] += 1
        self.cache.note_decode_step(slots)
        return logits[:rows]

    @torch.inference_mode()
    def decode_greedy(self, tokens: torch.Tensor, *, slots: Sequence[int], positions: torch.Tensor,
                      steps: int) -> torch.Tensor:
        """`steps` captured decode steps with the greedy sampler on the device and no host read in
        between: step i feeds the token step i - 1 chose.  tokens / positions [rows, 1] as for
        `decode`; returns the chosen tokens, int64 [steps, rows] (the same tokens `decode` followed
        by an argmax of its logits gives, step by step)."""
        rows = len(slots)
        if isinstance(steps, bool) or not isinstance(steps, int) or not 1 <= steps <= self.GREEDY_HISTORY_STEPS:
            raise ValueError(f"steps must be an integer in [1, {self.GREEDY_HISTORY_STEPS}]")
        self._check_pairs()
        width = next((w for w in sorted(self._graphs) if w >= rows), None)
        if width is None:
            raise RuntimeError("decode_greedy needs a captured graph of this width: call capture() first")
        self.cache.require_room(slots, steps)
        graph, graph_tokens, graph_positions, _ = self._graphs[width]
        history, cursors, _ = self._greedy[width]
        graph_tokens[:rows].copy_(tokens)
        graph_positions[:rows].copy_(positions)
        cursors.zero_()
        state = (width, tuple(slots))
        if state != self._decode_state:
            padded_slots = list(slots) + [0] * (width - rows)
            self.cache.set_decode_execution_state(
                slot_ids=torch.tensor(padded_slots, dtype=torch.int32, device=self.device),
                active_mask=torch.tensor([True] * rows + [False] * (width - rows), device=self.device))
            self._decode_state = state
        for _ in range(steps):
            graph.replay()
            self.cache.note_decode_step(slots)
        self.graph_replay_counts[width] += steps
        return history[:steps, :rows].clone()
