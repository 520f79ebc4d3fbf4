"""One decode step of a W4A4KV4 Llama with the glue between its packed kernels fused away.

The reference runs the Hugging Face module graph for a decode step: per layer about thirty
small tensor kernels (residual adds, LlamaRMSNorm, rotary embedding, SiLU and multiply,
Hadamard passes) surround the packed linears and the NQKV attention
(nestquant/models/fused_linear.py:276-421, nestquant/runtime/nqkv_batched_hf_backend.py:357-631).
Here the same arithmetic, in the same BF16 tensor-operation rounding, runs in nine launches
per layer:

    residual add + RMSNorm + Hadamard + A4 encode      nq_fused_input_stage (mode 1)
    q_proj, k_proj, v_proj                             nq_w4a4_gemv_grouped
    RoPE + Hadamard of q and k, KV append / page pack,
      paged attention, stage 1                         nq_nqkv_append_attention_decode (no output given)
    attention stage 2 + Hadamard + A4 encode           nq_attention_output_stage
    o_proj                                             nq_w4a4_gemv
    residual add + RMSNorm + Hadamard + A4 encode      nq_fused_input_stage (mode 1)
    gate_proj, up_proj                                 nq_w4a4_gemv_grouped
    SiLU(gate) * up + Hadamard + A4 encode             nq_fused_input_stage (mode 2)
    down_proj                                          nq_w4a4_gemv

preceded by one launch that advances the cache's tables and gathers the embedding and rotary
rows (nq_decode_step_begin) and followed by the LM head of up to 16 rows as one stream over its
BF16 weight (nq_bf16_rows_linear).

FusedLlamaPrefillStep runs a prompt (or a chunk of one) the same way over [rows * tokens]
activation rows: the input stages and linears as above (the linears on the matrix cores), RoPE
and Hadamard of queries and keys in one launch each, the KV writer, and the attention the
module graph would use (PyTorch's SDPA over the rotated BF16 keys and values of the chunk, or
the packed-cache kernel for a continuation).  The module graph stays the path for models these
steps do not recognise.
"""

from __future__ import annotations

import torch

import torch.nn.functional as F

from .nqkv import attention_output_stage, nqkv_prefill_attention
from .w4a4_linear import (BF16_ROWS_LINEAR_K, MATRIX_CORE_GEMV_ROWS, PreparedNQRTLinear, StageLinearSync, _gemm, _gemv,
                          bf16_rows_linear, bf16_rows_linear_grouped, can_use_bf16_rows_linear, can_use_fused_stage_linear,
                          decode_weight_bf16, can_use_w4a4_gemm_grouped, fused_input_stage, fused_stage_linear,
                          linear_packed_w4a4_gemm_grouped, linear_packed_w4a4_gemv_grouped, quantize_activation_cuda,
                          rope_hadamard_pair_cuda)


class UnsupportedForFusedDecode(ValueError):
    pass


def _require(condition: bool, reason: str) -> None:
    if not condition:
        raise UnsupportedForFusedDecode(reason)


class FusedLlamaDecodeStep:
    """Callable `(tokens [rows, 1], positions [rows, 1]) -> logits [rows, 1, vocab]` over a
    LlamaForCausalLM whose projections are FusedNQRTLinear modules and a BatchedNQKVLlamaCache.
    Raises UnsupportedForFusedDecode at construction for anything else."""

    # Which (input stage, linear) pairs of a layer run as one launch (`fused_stage_linear`): the linear's
    # workgroups decode their weights while the stage's few workgroups are still encoding.  Measured per
    # pair inside a launch sequence with cold weights (microseconds, two launches -> one, at 1 / 8 rows):
    # gate and up 24.0 -> 18.1 / 24.1 -> 20.4, down_proj 21.0 -> 16.5 / 23.6 -> 21.8, q, k and v
    # 11.8 -> 10.7 / 13.3 -> 12.7, o_proj 10.4 -> 10.2 / 12.2 -> 11.3.
    STAGE_LINEAR_PAIRS = frozenset({"qkv", "o", "gate_up", "down"})

    def __init__(self, model: torch.nn.Module, cache, *, expand_weights: bool = False,
                 stage_linear_pairs=None) -> None:
        """`expand_weights`: keep, beside every packed projection, the BF16 values its kernels
        multiply by (16 bits per weight in HBM instead of 6) and stream those for steps of up to
        16 rows: the same products without the per-step decode, which is what bounds the packed
        kernels.  The container on disk and the prefill path are unchanged.
        `stage_linear_pairs`: the pairs that run as one launch (a subset of STAGE_LINEAR_PAIRS, all of
        them when None, none when empty); same logits bit for bit either way."""
        from ..models.fused_linear import FusedNQRTLinear

        inner = getattr(model, "model", None)
        _require(inner is not None and hasattr(inner, "layers") and hasattr(model, "lm_head"),
                 "not a causal Llama model")
        _require(all(hasattr(inner, name) for name in ("embed_tokens", "rotary_emb", "norm")), "not a Llama body")
        self.model, self.inner, self.cache = model, inner, cache
        self.layers = []
        betas = None
        for layer in inner.layers:
            attention, mlp = getattr(layer, "self_attn", None), getattr(layer, "mlp", None)
            _require(attention is not None and mlp is not None, "layer without self_attn / mlp")
            _require(getattr(getattr(mlp, "act_fn", None), "__class__", type(None)).__name__ in {"SiLUActivation", "SiLU"},
                     "MLP activation is not SiLU")
            linears = [getattr(attention, n, None) for n in ("q_proj", "k_proj", "v_proj", "o_proj")]
            linears += [getattr(mlp, n, None) for n in ("gate_proj", "up_proj", "down_proj")]
            for linear in linears:
                _require(isinstance(linear, FusedNQRTLinear), "projection is not a FusedNQRTLinear")
                _require(linear.bias is None and linear.input_hadamard and linear.activation_q == 14
                         and not linear.force_w4a4_tiled_fallback and len(linear.activation_betas) == 4,
                         "projection configuration outside the fused step")
                _require(betas is None or linear.activation_betas == betas, "projections disagree on activation betas")
                betas = linear.activation_betas
            for norm in (layer.input_layernorm, layer.post_attention_layernorm):
                _require(hasattr(norm, "weight") and hasattr(norm, "variance_epsilon"), "norm is not an RMSNorm")
            self.layers.append((layer, attention, mlp, linears))
        _require(len(self.layers) == cache.num_layers, "layer count disagrees with the cache")
        hidden = inner.embed_tokens.weight.shape[1]
        _require(hidden & (hidden - 1) == 0 and hidden % 32 == 0, "hidden size is not a power of two")
        self.hidden = hidden
        self._rope_tables: torch.Tensor | None = None
        self.expand_weights = bool(expand_weights)
        self._expanded: dict[int, tuple] = {}
        self._weights: dict[int, tuple] = {}
        pairs = self.STAGE_LINEAR_PAIRS if stage_linear_pairs is None else frozenset(stage_linear_pairs)
        if not pairs <= self.STAGE_LINEAR_PAIRS:
            raise ValueError(f"stage_linear_pairs must be a subset of {sorted(self.STAGE_LINEAR_PAIRS)}")
        self.stage_linear_pairs = pairs
        self._pair_sync: StageLinearSync | None = None

    # -- stage + linear as one launch -------------------------------------------------------------
    def pairs_failed(self) -> bool:
        """Whether a consumer of some earlier one-launch pair gave up its bounded wait (its outputs were
        then not stored).  Reads a word of pinned host memory: no synchronisation."""
        return self._pair_sync is not None and self._pair_sync.timed_out

    def disable_pairs(self) -> None:
        """Back to two launches per pair for good (after `pairs_failed`); call with the stream idle."""
        self.stage_linear_pairs = frozenset()
        if self._pair_sync is not None:
            self._pair_sync.reset()

    def _pair(self, name: str, rows: int, k: int, weights) -> bool:
        return name in self.stage_linear_pairs and can_use_fused_stage_linear(rows, k, weights)

    def _rope(self, embedded: torch.Tensor, positions: torch.Tensor, *, padded: bool = False
              ) -> tuple[torch.Tensor, torch.Tensor]:
        """BF16 (cos, sin) [positions.numel(), head_dim] of the model's rotary embedding.  For
        embeddings that depend on the position alone the module is evaluated once, over every
        position the cache can hold, and a step gathers its rows (one launch instead of the
        module's dozen)."""
        rotary = self.inner.rotary_emb
        if getattr(rotary, "rope_type", "default") not in ("default", "llama3", "linear"):
            cos, sin = rotary(embedded, positions)
            dim = cos.shape[-1]
            return cos.to(torch.bfloat16).reshape(-1, dim).contiguous(), sin.to(torch.bfloat16).reshape(-1, dim).contiguous()
        if self._rope_tables is None:
            every = torch.arange(self.cache.max_cache_len, device=embedded.device)[None, :]
            cos, sin = rotary(embedded[:1, :1], every)
            self._rope_tables = torch.stack((cos[0], sin[0])).to(torch.bfloat16).contiguous()     # [2, positions, dim]
        index = positions.reshape(-1)
        if padded:                      # positions of padding tokens may lie past the cache's last one
            index = index.clamp(max=self._rope_tables.shape[1] - 1)
        both = self._rope_tables.index_select(1, index)
        return both[0], both[1]

    @staticmethod
    def _prepared(linear, device) -> PreparedNQRTLinear:
        prepared = linear._prepared_for(device)
        _require(prepared.resolved_words is not None, "weight has no resolved form")
        return prepared

    def _layer_weights(self, index: int, device) -> tuple[PreparedNQRTLinear, ...]:
        """The seven prepared projections of layer `index` (q, k, v, o, gate, up, down), looked up once
        and kept while the modules still hold them on this device."""
        linears = self.layers[index][3]
        kept = self._weights.get(index)
        if (kept is None or kept[0].device != device
                or not all(weight is linear._prepared for weight, linear in zip(kept, linears))):
            kept = self._weights[index] = tuple(self._prepared(linear, device) for linear in linears)
        return kept

    @staticmethod
    def _gemv_rows(activation) -> int:
        return MATRIX_CORE_GEMV_ROWS if activation.feature_count % 128 == 0 else 8

    def _linear(self, activation, prepared: PreparedNQRTLinear) -> torch.Tensor:
        if activation.token_count <= self._gemv_rows(activation):
            return _gemv(activation, prepared, split_k=0, output_dtype=torch.bfloat16)
        return _gemm(activation, prepared, output_dtype=torch.bfloat16)

    def _linears(self, activation, prepared: list[PreparedNQRTLinear]) -> list[torch.Tensor]:
        if activation.token_count <= self._gemv_rows(activation):
            return linear_packed_w4a4_gemv_grouped(activation, prepared, output_dtype=torch.bfloat16)
        if can_use_w4a4_gemm_grouped(activation, prepared):      # a long prefill: one product for the group
            return linear_packed_w4a4_gemm_grouped(activation, prepared, checked=True)
        return [self._linear(activation, weight) for weight in prepared]

    def _expanded_layer(self, index: int, device) -> tuple | None:
        """(q|k|v rows, their sizes, o, gate|up rows, their sizes, down) of layer `index` as BF16
        [N, K] tensors, decoded once; None when a projection's K is not one the stream kernel takes."""
        if index not in self._expanded:
            prepared = [self._prepared(linear, device) for linear in self.layers[index][3]]
            if any(weight.record.feature_count not in BF16_ROWS_LINEAR_K for weight in prepared):
                self._expanded[index] = None
            else:
                q, k, v, o, gate, up, down = (decode_weight_bf16(weight) for weight in prepared)
                self._expanded[index] = (torch.cat((q, k, v)), [q.shape[0], k.shape[0], v.shape[0]], o,
                                         torch.cat((gate, up)), [gate.shape[0], up.shape[0]], down)
        return self._expanded[index]

    def _table_rope(self) -> bool:
        return getattr(self.inner.rotary_emb, "rope_type", "default") in ("default", "llama3", "linear")

    @torch.inference_mode()
    def __call__(self, tokens: torch.Tensor, positions: torch.Tensor, *, advance: bool = False) -> torch.Tensor:
        """`advance`: the step itself advances the cache's tables by one token per active row
        (`BatchedNQKVLlamaCache.begin_decode_step`, which the caller has otherwise done), in the
        launch that also gathers the embedding and rotary rows when the model allows it."""
        cache, inner = self.cache, self.inner
        manager = cache.manager
        rows = tokens.shape[0]
        if tokens.shape != (rows, 1) or positions.shape != (rows, 1) or rows != cache._rows:
            raise ValueError("the fused decode step takes [rows, 1] tokens and positions for the rows in flight")
        device = tokens.device
        table = inner.embed_tokens.weight
        if table.dtype != torch.bfloat16:
            raise TypeError("the fused decode step runs BF16 models")
        if (advance and self._table_rope() and type(inner.embed_tokens) is torch.nn.Embedding
                and table.is_contiguous() and table.shape[1] % 8 == 0 and tokens.is_contiguous()
                and positions.is_contiguous() and tokens.dtype == positions.dtype == torch.int64):
            if self._rope_tables is None:
                self._rope(torch.empty((1, 1, self.hidden), dtype=torch.bfloat16, device=device), positions)
            embedded, query_rope = manager.begin_decode_step(rows=rows, tokens=tokens, embedding=table,
                                                             positions=positions, rotary=self._rope_tables)
        else:
            if advance:
                cache.begin_decode_step()
            embedded = inner.embed_tokens(tokens)                           # [rows, 1, hidden]
            query_rope = self._rope(embedded, positions)                    # 2 x [rows, head_dim]
        heads, kv_heads, dim = cache.num_query_heads, cache.num_kv_heads, cache.head_dim
        workspace = cache._workspace(rows, torch.bfloat16)

        sync = None
        if self.stage_linear_pairs and not (self.expand_weights and rows <= 16):
            if self._pair_sync is None:
                self._pair_sync = StageLinearSync(device, sets=4 * len(self.layers))
            sync = self._pair_sync
            sync.begin_step()
        delta, residual = embedded.view(rows, self.hidden), None
        for index, (layer, attention, mlp, linears) in enumerate(self.layers):
            q_w, k_w, v_w, o_w, gate_w, up_w, down_w = self._layer_weights(index, device)
            table = linears[0].activation_beta_table
            expanded = self._expanded_layer(index, device) if self.expand_weights and rows <= 16 else None
            if sync is not None and expanded is None and self._pair("qkv", rows, self.hidden, [q_w, k_w, v_w]):
                (query, key, value), _, residual, _ = fused_stage_linear(
                    delta, [q_w, k_w, v_w], sync, mode="rmsnorm", residual=residual, norm_weight=layer.input_layernorm.weight,
                    eps=layer.input_layernorm.variance_epsilon, beta_table=table, want_residual=True)
            else:
                activation, residual, _ = fused_input_stage(
                    delta, mode="rmsnorm", residual=residual, norm_weight=layer.input_layernorm.weight,
                    eps=layer.input_layernorm.variance_epsilon, beta_table=table, want_residual=True)
                if expanded is not None:
                    query, key, value = bf16_rows_linear_grouped(activation.decoded, expanded[0], expanded[1])
                else:
                    query, key, value = self._linears(activation, [q_w, k_w, v_w])
            # the new token joins the cache inside the attention launch, which leaves per-chunk results;
            # o_proj's input stage merges them as it loads its rows
            manager.append_and_attend(
                index, query.view(rows, heads, dim), key.view(rows, kv_heads, dim), value.view(rows, kv_heads, dim),
                attention_scale=float(attention.scaling), workspace=workspace, rotate=True, rope=query_rope,
                merge=False)
            if sync is not None and expanded is None and self._pair("o", rows, heads * dim, [o_w]):
                (delta,), _, _, _ = fused_stage_linear(None, [o_w], sync, mode="attention", beta_table=table,
                                                       attention_workspace=workspace)
            else:
                o_input, _ = attention_output_stage(workspace, q=14, beta_table=table, hadamard=True)
                delta = self._linear(o_input, o_w) if expanded is None else bf16_rows_linear(o_input.decoded, expanded[2])
            if sync is not None and expanded is None and self._pair("gate_up", rows, self.hidden, [gate_w, up_w]):
                (gate, up), _, residual, _ = fused_stage_linear(
                    delta, [gate_w, up_w], sync, mode="rmsnorm", residual=residual,
                    norm_weight=layer.post_attention_layernorm.weight, eps=layer.post_attention_layernorm.variance_epsilon,
                    beta_table=table, want_residual=True)
            else:
                activation, residual, _ = fused_input_stage(
                    delta, mode="rmsnorm", residual=residual, norm_weight=layer.post_attention_layernorm.weight,
                    eps=layer.post_attention_layernorm.variance_epsilon, beta_table=table, want_residual=True)
                if expanded is not None:
                    gate, up = bf16_rows_linear_grouped(activation.decoded, expanded[3], expanded[4])
                else:
                    gate, up = self._linears(activation, [gate_w, up_w])
            if sync is not None and expanded is None and self._pair("down", rows, up.shape[-1], [down_w]):
                (delta,), _, _, _ = fused_stage_linear(up, [down_w], sync, mode="swiglu", gate=gate, beta_table=table)
            else:
                activation, _, _ = fused_input_stage(up, mode="swiglu", gate=gate, beta_table=table)
                delta = (self._linear(activation, down_w) if expanded is None
                         else bf16_rows_linear(activation.decoded, expanded[5]))
        _, _, normed = fused_input_stage(delta, mode="rmsnorm", residual=residual, norm_weight=inner.norm.weight,
                                         eps=inner.norm.variance_epsilon, encode=False, want_staged=True)
        return self._lm_head(normed.view(rows, self.hidden)).view(rows, 1, -1)

    def _lm_head(self, normed: torch.Tensor) -> torch.Tensor:
        """Logits of a few rows: one stream over the BF16 head weight when it has the shape the
        stream kernel takes, the module's own linear otherwise."""
        head = self.model.lm_head
        if getattr(head, "bias", None) is None and can_use_bf16_rows_linear(normed, head.weight):
            return bf16_rows_linear(normed, head.weight)
        return head(normed)


class FusedLlamaPrefillStep(FusedLlamaDecodeStep):
    """Callable `(tokens [rows, width], positions [rows, width]) -> logits [rows, width, vocab]`
    for the rows `BatchedNQKVLlamaCache.set_batch_state` has announced; same model requirements
    as FusedLlamaDecodeStep."""

    @torch.inference_mode()
    def __call__(self, tokens: torch.Tensor, positions: torch.Tensor, *,
                 keep: torch.Tensor | None = None) -> torch.Tensor:
        """`keep` (int64 [rows], optional): the one token of every row whose logits are wanted;
        the final norm and the LM head then run on those rows only and the result is
        [rows, 1, vocab]."""
        cache, inner = self.cache, self.inner
        manager = cache.manager
        rows, width = tokens.shape
        if positions.shape != (rows, width) or rows != cache._rows:
            raise ValueError("the fused prefill step takes [rows, width] tokens and positions for the rows in flight")
        if keep is not None and (keep.shape != (rows,) or keep.dtype != torch.int64 or keep.device != tokens.device):
            raise ValueError("keep holds one int64 token index per row, on the tokens' device")
        device = tokens.device
        embedded = inner.embed_tokens(tokens)                               # [rows, width, hidden]
        if embedded.dtype != torch.bfloat16:
            raise TypeError("the fused prefill step runs BF16 models")
        count = rows * width
        heads, kv_heads, dim = cache.num_query_heads, cache.num_kv_heads, cache.head_dim
        rope = self._rope(embedded, positions, padded=True)                 # 2 x [rows * width, head_dim]
        over_cache = cache.packed_prefill or cache._continuation

        delta, residual = embedded.reshape(count, self.hidden), None
        for index, (layer, attention, mlp, linears) in enumerate(self.layers):
            q_w, k_w, v_w, o_w, gate_w, up_w, down_w = self._layer_weights(index, device)
            table = linears[0].activation_beta_table
            activation, residual, _ = fused_input_stage(
                delta, mode="rmsnorm", residual=residual, norm_weight=layer.input_layernorm.weight,
                eps=layer.input_layernorm.variance_epsilon, beta_table=table, want_residual=True)
            query, key, value = self._linears(activation, [q_w, k_w, v_w])
            query, key = rope_hadamard_pair_cuda(query.view(count, heads, dim), key.view(count, kv_heads, dim), rope=rope)
            query, key = query.view(rows, width, heads, dim), key.view(rows, width, kv_heads, dim)
            value = value.view(rows, width, kv_heads, dim)
            manager.write_layer(index, key, value)
            scale = float(attention.scaling)
            if over_cache:
                attended = nqkv_prefill_attention(query, manager.layers[index], slot_ids=manager.step_slot_ids,
                                                  active_mask=manager.step_active, counts=manager.step_counts, scale=scale)
            else:
                attended = F.scaled_dot_product_attention(
                    query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2), dropout_p=0.0, is_causal=True,
                    scale=scale, enable_gqa=heads != kv_heads).transpose(1, 2)
            o_input = quantize_activation_cuda(attended.reshape(count, heads * dim), q=14,
                                               betas=linears[3].activation_betas, beta_table=table, hadamard=True)
            delta = self._linear(o_input, o_w)
            activation, residual, _ = fused_input_stage(
                delta, mode="rmsnorm", residual=residual, norm_weight=layer.post_attention_layernorm.weight,
                eps=layer.post_attention_layernorm.variance_epsilon, beta_table=table, want_residual=True)
            gate, up = self._linears(activation, [gate_w, up_w])
            activation, _, _ = fused_input_stage(up, mode="swiglu", gate=gate, beta_table=table)
            delta = self._linear(activation, down_w)
        if keep is not None:
            flat = torch.arange(rows, device=device) * width + keep
            delta, residual = delta.index_select(0, flat), residual.index_select(0, flat)
        _, _, normed = fused_input_stage(delta, mode="rmsnorm", residual=residual, norm_weight=inner.norm.weight,
                                         eps=inner.norm.variance_epsilon, encode=False, want_staged=True)
        if keep is not None:
            return self._lm_head(normed.view(rows, self.hidden)).view(rows, 1, -1)
        return self.model.lm_head(normed.view(rows, width, self.hidden))
