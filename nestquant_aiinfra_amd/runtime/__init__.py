"""Operators of the packed W4A4KV4 path, under the names the reference exports from
nestquant.runtime (nestquant/runtime/__init__.py) for this path, plus the fused steps."""

from __future__ import annotations

import importlib

_EXPORTS = {
    "PreparedNQA4Activation": "w4a4_linear",
    "PreparedNQRTLinear": "w4a4_linear",
    "quantize_rows_packed": "w4a4_linear",
    "hadamard_cuda": "w4a4_linear",
    "rope_hadamard_cuda": "w4a4_linear",
    "rope_hadamard_pair_cuda": "w4a4_linear",
    "quantize_activation_cuda": "w4a4_linear",
    "fused_input_stage": "w4a4_linear",
    "quantize_weight_nqrt4": "w4a4_linear",
    "StageLinearSync": "w4a4_linear",
    "can_use_fused_stage_linear": "w4a4_linear",
    "fused_stage_linear": "w4a4_linear",
    "resolve_weight": "w4a4_linear",
    "prepare_fused_linear": "w4a4_linear",
    "dequantize_rows_packed": "w4a4_linear",
    "dequantize_record": "w4a4_linear",
    "decode_packed_a4": "w4a4_linear",
    "can_use_w4a4_gemv_m1": "w4a4_linear",
    "can_use_w4a4_mma_small_m": "w4a4_linear",
    "can_use_w4a4_mma_m16": "w4a4_linear",
    "can_use_w4a4_mma_large_m_staged": "w4a4_linear",
    "can_use_w4a4_mma_m128_staged": "w4a4_linear",
    "can_use_w4a4_mma_chunked_staged": "w4a4_linear",
    "linear_packed_w4a4_gemv_grouped": "w4a4_linear",
    "can_use_w4a4_gemm_grouped": "w4a4_linear",
    "linear_packed_w4a4_gemm_grouped": "w4a4_linear",
    "linear_packed_w4a4_gemv_m1": "w4a4_linear",
    "linear_packed_w4a4_gemv_m1_fp32_probe": "w4a4_linear",
    "linear_packed_w4a4_gemv_m1_splitk_probe": "w4a4_linear",
    "linear_packed_w4a4_gemv_m1_splitk_fp32_probe": "w4a4_linear",
    "linear_packed_w4a4_mma_small_m": "w4a4_linear",
    "linear_packed_w4a4_mma_small_m_splitk_probe": "w4a4_linear",
    "decode_weight_bf16": "w4a4_linear",
    "can_use_bf16_rows_linear": "w4a4_linear",
    "bf16_rows_linear": "w4a4_linear",
    "bf16_rows_linear_grouped": "w4a4_linear",
    "linear_packed_w4a4_mma_m16": "w4a4_linear",
    "linear_packed_w4a4_mma_large_m_staged": "w4a4_linear",
    "linear_packed_w4a4_mma_m128_staged": "w4a4_linear",
    "linear_packed_w4a4_mma_chunked_staged": "w4a4_linear",
    "linear_packed_w4a4_mma_chunked_staged_probe": "w4a4_linear",
    "slice_pad_packed_activation_rows": "w4a4_linear",
    "PreparedNQKVPage": "nqkv",
    "quantize_nqkv_page_cuda": "nqkv",
    "dequantize_nqkv_page": "nqkv",
    "dequantize_nqkv_page_triton": "nqkv",
    "NQKVPageHandle": "nqkv",
    "NQKVPagePool": "nqkv",
    "BatchedNQKVMetadata": "nqkv",
    "NQKVHotColdCache": "nqkv",
    "BatchedNQKVAttentionWorkspace": "nqkv",
    "launch_nqkv_decode_attention": "nqkv",
    "attention_output_stage": "nqkv",
    "nqkv_decode_attention_batched_k1": "nqkv",
    "nqkv_prefill_attention": "nqkv",
    "BatchedNQKVCacheManager": "nqkv",
    "append_hot_k1_graph_safe": "nqkv",
    "launch_pack_full_hot_pages_graph_safe": "nqkv",
    "PagedNQKVCache": "nqkv_single",
    "NQKVAttentionWorkspace": "nqkv_single",
    "nqkv_decode_attention_k1": "nqkv_single",
    "NQKVLlamaCache": "nqkv_single",
    "install_nqkv_llama_backend": "nqkv_single",
    "cuda_e8_available": "cuda_e8",
    "e8_nearest_cuda": "cuda_e8",
    "bf16_gemm": "w4a4_linear",
    "BatchedNQKVLlamaCache": "nqkv_hf_backend",
    "install_batched_nqkv_llama_backend": "nqkv_hf_backend",
    "greedy_sample_": "nqkv_hf_backend",
    "greedy_sample_workspace": "nqkv_hf_backend",
    "BatchedNQKVLlamaRunner": "nqkv_hf_backend",
    "RequestStatus": "continuous_batching",
    "DecodeRequest": "continuous_batching",
    "ContinuousBatchScheduler": "continuous_batching",
    "RaggedDecodeBackend": "inference_engine",
    "EngineStep": "inference_engine",
    "AdmissionPolicy": "inference_engine",
    "GreedyHostSampler": "inference_engine",
    "ContinuousBatchInferenceEngine": "inference_engine",
    "UnsupportedForFusedDecode": "llama_decode_step",
    "FusedLlamaDecodeStep": "llama_decode_step",
    "FusedLlamaPrefillStep": "llama_decode_step",
}

__all__ = sorted(_EXPORTS)


def __getattr__(name: str):
    # resolved on first use: importing the package does not import torch, transformers or the library
    module = _EXPORTS.get(name)
    if module is None:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
    value = getattr(importlib.import_module(f"{__name__}.{module}"), name)
    globals()[name] = value
    return value


def __dir__():
    return sorted(set(globals()) | set(_EXPORTS))
