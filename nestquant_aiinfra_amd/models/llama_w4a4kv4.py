"""Assembly of a W4A4KV4 Llama: quantise a model's projections into an NQMC file, swap them
for FusedNQRTLinear modules and attach the batched NQKV cache.  Follows the offline flow of
nestquant/core/quantizer.py:214-301 + nestquant/core/tensor_checkpoint.py:59-118 (done on the
GPU here) and the assembly of scripts/serve_w4a4kv4.py:118-177."""

from __future__ import annotations

from pathlib import Path
from typing import Sequence

import torch
from torch import nn

from ..core.model_checkpoint import PAPER_HADAMARD_FORMAT, NQMCFileReader, write_nqmc
from ..core.rotation import hadamard
from ..runtime.nqkv_hf_backend import BatchedNQKVLlamaCache, BatchedNQKVLlamaRunner, install_batched_nqkv_llama_backend
from ..runtime.w4a4_linear import quantize_weight_nqrt4
from .fused_linear import convert_linears_to_fused_nqrt_

PROJECTIONS = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")
ACTIVATION_BETAS = tuple(value / 14 for value in (3.47, 4.74, 6.90, 18.11))
WEIGHT_BETAS = tuple(value / 14 for value in (4.0, 5.5, 7.0, 18.0))
KEY_BETAS = tuple(value / 14 for value in (3.50, 4.58, 6.47, 17.06))
VALUE_BETAS = tuple(value / 14 for value in (3.53, 5.59, 9.62, 29.03))


def projection_names(model: nn.Module) -> list[str]:
    return [name for name, module in model.named_modules()
            if isinstance(module, nn.Linear) and name.rsplit(".", 1)[-1] in PROJECTIONS]


@torch.inference_mode()
def write_w4_checkpoint(model: nn.Module, path: str | Path, *, betas: Sequence[float] = WEIGHT_BETAS,
                        q: int = 14, first_dither_seed: int = 20261101) -> list[str]:
    """Rotate every projection weight along its input axis, quantise it to NQRT4 on the GPU
    (independent E8 blocks, stateless dither, one seed per tensor) and write an NQMC file that
    also holds the remaining dense tensors.  Returns the converted module names."""
    names = projection_names(model)
    quantized = {}
    for index, name in enumerate(names):
        weight = dict(model.named_modules())[name].weight
        rotated = hadamard(weight.detach().float())
        quantized[f"{name}.weight"] = quantize_weight_nqrt4(
            rotated, q=q, betas=betas, dither_seed=first_dither_seed + index, tensor_name=f"{name}.weight")
    state = model.state_dict()
    dense, aliases, seen = {}, {}, {}
    for key, tensor in state.items():
        if key in quantized:
            continue
        pointer = (tensor.data_ptr(), tuple(tensor.shape))
        if pointer in seen:
            aliases[key] = seen[pointer]
            continue
        seen[pointer] = key
        dense[key] = tensor.detach().cpu()
    write_nqmc(path, dense_tensors=dense, quantized_tensors=quantized, aliases=aliases, model_metadata={
        "hadamard_rotation": {"format": PAPER_HADAMARD_FORMAT, "converted_linear_names": names}})
    return names


def build_w4a4kv4_runner(model: nn.Module, checkpoint: str | Path, *, capacity: int, max_cache_len: int,
                         page_size: int = 16, activation_betas: Sequence[float] = ACTIVATION_BETAS,
                         key_betas: Sequence[float] = KEY_BETAS, value_betas: Sequence[float] = VALUE_BETAS,
                         enable_m1_down_splitk: bool = False,
                         fused_decode: bool | None = None, fused_prefill: bool | None = None,
                         packed_prefill: bool = False, expand_weights: bool = False,
                         stage_linear_pairs=None, decode_hints: bool = True) -> BatchedNQKVLlamaRunner:
    """Swap the projections of `model` (BF16, on the GPU, eval mode) for packed W4A4 modules
    read from `checkpoint` and attach a batched NQKV4 cache; returns the runner."""
    reader = NQMCFileReader(checkpoint)
    names = [name for name in projection_names(model)]
    convert_linears_to_fused_nqrt_(model, reader, names, compute_backend="packed_w4a4_cuda_mma", activation_q=14,
                                   activation_betas=tuple(activation_betas),
                                   enable_m1_down_splitk=enable_m1_down_splitk)
    return attach_w4a4kv4_cache(model, capacity=capacity, max_cache_len=max_cache_len, page_size=page_size,
                                key_betas=key_betas, value_betas=value_betas, fused_decode=fused_decode,
                                fused_prefill=fused_prefill, packed_prefill=packed_prefill,
                                expand_weights=expand_weights, stage_linear_pairs=stage_linear_pairs,
                                decode_hints=decode_hints)


def attach_w4a4kv4_cache(model: nn.Module, *, capacity: int, max_cache_len: int, page_size: int = 16,
                         key_betas: Sequence[float] = KEY_BETAS, value_betas: Sequence[float] = VALUE_BETAS,
                         fused_decode: bool | None = None, fused_prefill: bool | None = None,
                         packed_prefill: bool = False, expand_weights: bool = False,
                         stage_linear_pairs=None, decode_hints: bool = True) -> BatchedNQKVLlamaRunner:
    """A batched NQKV4 cache of `capacity` slots and its runner over a model whose projections are
    already packed modules (an engine of another capacity over the same weights: the packed weights
    are shared, the attention modules point at the newest cache).  `decode_hints`: the page pools keep
    four more bits per block so that the attention kernels skip the lattice searches of the KV decode
    (same outputs bit for bit; 10.5 % more pool memory)."""
    config = model.config
    head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
    device = next(model.parameters()).device
    cache = BatchedNQKVLlamaCache(
        capacity=capacity, num_layers=config.num_hidden_layers, num_query_heads=config.num_attention_heads,
        num_kv_heads=config.num_key_value_heads, head_dim=head_dim, max_cache_len=max_cache_len,
        page_size=page_size, q=14, key_betas=key_betas, value_betas=value_betas, dtype=torch.bfloat16, device=device,
        packed_prefill=packed_prefill, decode_hints=decode_hints)
    install_batched_nqkv_llama_backend(model, cache)
    return BatchedNQKVLlamaRunner(model, cache, fused_decode=fused_decode, fused_prefill=fused_prefill,
                                  expand_weights=expand_weights, stage_linear_pairs=stage_linear_pairs)
