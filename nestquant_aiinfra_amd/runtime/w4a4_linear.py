"""Packed W4A4 operators: NQA4 activation encoder, NQRT4 weight preparation, and the
linear kernels that consume both without ever materialising a BF16 matrix.

Names, argument meaning and error behaviour mirror the reference's Python surface:
  quantize_activation_cuda / PreparedNQA4Activation   nestquant/runtime/triton_w4a4_linear.py:489-617
  prepare_fused_linear / PreparedNQRTLinear           nestquant/runtime/triton_fused_linear.py:135-165
  can_use_w4a4_* / linear_packed_w4a4_*               nestquant/runtime/cuda_w4a4_mma.py:44-619
Every operator calls the HIP library through its C ABI; there is no other compute path.
"""

from __future__ import annotations

import ctypes
import math
import weakref
from dataclasses import dataclass
from typing import Any, Sequence

import torch

from .. import _native
from ..core.codec import STATELESS_DITHER_ALGORITHM, UPSTREAM_CODEC_SEMANTICS
from ..core.packing import PackedNestQuantIndices, bits_for_cardinality
from ..core.tensor_checkpoint import PackedNestQuantTensor


# --------------------------------------------------------------------------------------
# containers
# --------------------------------------------------------------------------------------

@dataclass(frozen=True)
class PreparedNQA4Activation:
    """GPU-resident packed activation rows consumed without BF16 expansion."""

    code_payload: torch.Tensor
    beta_payload: torch.Tensor
    row_norms: torch.Tensor
    beta_table: torch.Tensor
    original_shape: tuple[int, ...]
    q: int
    code_width: int
    beta_width: int
    output_dtype: torch.dtype
    # BF16 [tokens, features] decode of the payloads, emitted by the encoder as a side
    # product so that the linear kernels need not decode the activation again; None for
    # activations assembled from payloads alone (the kernels then decode them once per call).
    decoded: torch.Tensor | None = None

    @property
    def token_count(self) -> int:
        return math.prod(self.original_shape[:-1])

    @property
    def feature_count(self) -> int:
        return self.original_shape[-1]

    @property
    def resident_bytes(self) -> int:
        return sum(t.numel() * t.element_size()
                   for t in (self.code_payload, self.beta_payload, self.row_norms, self.beta_table))


@dataclass(frozen=True)
class PreparedNQRTLinear:
    """GPU-resident packed streams and metadata of one NQRT4 weight."""

    record: Any          # PackedNestQuantTensor (ours or the reference's: same attributes)
    # The NQRT4 streams on the device, or None once the resolved form has replaced them (the record
    # still holds them on the host; `prepare_fused_linear(..., keep_streams=True)` keeps both).
    code_payload: torch.Tensor | None
    beta_payload: torch.Tensor | None
    row_norms: torch.Tensor
    beta_table: torch.Tensor
    # Optional resolved form (int32 word + int16 tail per 8-weight block): the lattice point
    # each block's decode lands on, found once here so that the linear kernels need neither
    # lattice search.  6 bits per weight instead of (or, with keep_streams, beside) the 4.25-bit streams.
    resolved_words: torch.Tensor | None = None
    resolved_tails: torch.Tensor | None = None

    @property
    def device(self) -> torch.device:
        return self.row_norms.device

    @property
    def resident_bytes(self) -> int:
        """Bytes of device memory this weight holds."""
        tensors = (self.code_payload, self.beta_payload, self.row_norms, self.beta_table, self.resolved_words,
                   self.resolved_tails)
        return sum(t.numel() * t.element_size() for t in tensors if t is not None)


# --------------------------------------------------------------------------------------
# encoders
# --------------------------------------------------------------------------------------

def _beta_values(betas: Sequence[float]) -> tuple[float, ...]:
    try:
        values = tuple(float(value) for value in betas)
    except (TypeError, ValueError) as error:
        raise TypeError("betas must be a nonempty sequence of numbers") from error
    if not values or any(not math.isfinite(value) or value <= 0 for value in values):
        raise ValueError("betas must be positive finite values")
    return values


def quantize_rows_packed(rows: torch.Tensor, *, q: int, beta_table: torch.Tensor,
                         dither_seed: int | None = None, block_offset: int = 0,
                         decoded: torch.Tensor | None = None, hadamard: bool = False
                         ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Encode ``rows`` [R, n] (float32 / bfloat16 / float16, on the GPU) into packed 4-bit
    codes, packed 2-bit beta ids and float32 row norms with one kernel launch.  ``decoded``
    (optional BF16 [R, n]) receives the decode of the stored codes."""
    device = _native.require_cuda(rows, beta_table)
    if rows.ndim != 2:
        raise ValueError("rows must have shape [rows, features]")
    count, n = rows.shape
    codes = torch.empty(count * n // 2, dtype=torch.uint8, device=device)
    beta_ids = torch.empty(count * n // 32, dtype=torch.uint8, device=device)
    norms = torch.empty(count, dtype=torch.float32, device=device)
    _native.check(_native.library().nq_quantize_rows(
        rows.data_ptr(), _native.dtype_tag(rows.dtype), count, n, q, beta_table.data_ptr(),
        beta_table.numel(), int(dither_seed is not None), int(dither_seed or 0), block_offset,
        int(hadamard), codes.data_ptr(), beta_ids.data_ptr(), norms.data_ptr(),
        None if decoded is None else decoded.data_ptr(), _native.stream_handle(device)))
    return codes, beta_ids, norms


def hadamard_cuda(inputs: torch.Tensor, *, compute_dtype: torch.dtype | None = None,
                  output_dtype: torch.dtype | None = None) -> torch.Tensor:
    """Normalized Hadamard transform along the last axis in one kernel.  `compute_dtype` is the
    dtype whose arithmetic the butterflies follow (default: the input's; float32 = no
    intermediate rounding); `output_dtype` defaults to the input's."""
    if not isinstance(inputs, torch.Tensor) or not inputs.is_floating_point() or inputs.ndim == 0:
        raise ValueError("expected a floating-point tensor with a feature axis")
    device = _native.require_cuda(inputs)
    n = inputs.shape[-1]
    out = torch.empty(inputs.shape, dtype=output_dtype or inputs.dtype, device=device)
    _native.check(_native.library().nq_hadamard(
        inputs.data_ptr(), _native.dtype_tag(inputs.dtype), inputs.numel() // n, n,
        _native.dtype_tag(compute_dtype or inputs.dtype), out.data_ptr(), _native.dtype_tag(out.dtype),
        _native.stream_handle(device)))
    return out


def rope_hadamard_cuda(vectors: torch.Tensor, *, rope: tuple[torch.Tensor, torch.Tensor] | None = None,
                       hadamard: bool = True) -> torch.Tensor:
    """Rotary embedding and / or Hadamard rotation of BF16 head vectors [rows, heads, head_dim]
    in one kernel: `rope` = BF16 (cos, sin) [rows, head_dim] applied as transformers'
    apply_rotary_pos_emb does in BF16, then ``hadamard(x.float()).to(bfloat16)``."""
    device = _native.require_cuda(vectors)
    if vectors.dtype != torch.bfloat16 or vectors.ndim != 3 or not vectors.is_contiguous():
        raise ValueError("expected a contiguous BF16 tensor [rows, heads, head_dim]")
    rows, heads, dim = vectors.shape
    if rope is not None:
        for table in rope:
            if table.dtype != torch.bfloat16 or tuple(table.shape) != (rows, dim) or not table.is_contiguous():
                raise ValueError("rotary tables must be contiguous BF16 [rows, head_dim]")
    out = torch.empty_like(vectors)
    _native.check(_native.library().nq_rope_hadamard(
        vectors.data_ptr(), rows, heads, dim, None if rope is None else rope[0].data_ptr(),
        None if rope is None else rope[1].data_ptr(), int(hadamard), out.data_ptr(), _native.stream_handle(device)))
    return out


def rope_hadamard_pair_cuda(query: torch.Tensor, key: torch.Tensor, *,
                            rope: tuple[torch.Tensor, torch.Tensor] | None = None, hadamard: bool = True
                            ) -> tuple[torch.Tensor, torch.Tensor]:
    """`rope_hadamard_cuda` of the queries [rows, query_heads, head_dim] and the keys [rows, key_heads,
    head_dim] of the same rows in one launch."""
    device = _native.require_cuda(query, key)
    for vectors in (query, key):
        if vectors.dtype != torch.bfloat16 or vectors.ndim != 3 or not vectors.is_contiguous():
            raise ValueError("expected contiguous BF16 tensors [rows, heads, head_dim]")
    rows, heads, dim = query.shape
    if key.shape[0] != rows or key.shape[2] != dim:
        raise ValueError("queries and keys must agree on rows and head_dim")
    if rope is not None:
        for table in rope:
            if table.dtype != torch.bfloat16 or tuple(table.shape) != (rows, dim) or not table.is_contiguous():
                raise ValueError("rotary tables must be contiguous BF16 [rows, head_dim]")
    query_out, key_out = torch.empty_like(query), torch.empty_like(key)
    _native.check(_native.library().nq_rope_hadamard_pair(
        query.data_ptr(), heads, query_out.data_ptr(), key.data_ptr(), key.shape[1], key_out.data_ptr(), rows, dim,
        None if rope is None else rope[0].data_ptr(), None if rope is None else rope[1].data_ptr(), int(hadamard),
        _native.stream_handle(device)))
    return query_out, key_out


def quantize_activation_cuda(inputs: torch.Tensor, *, q: int, betas: Sequence[float],
                             beta_table: torch.Tensor | None = None,
                             hadamard: bool = False) -> PreparedNQA4Activation:
    """Encode floating activations into packed NQA4 payloads on the GPU.

    `hadamard=True` (an extension) rotates the rows inside the same kernel, equivalent to
    encoding ``hadamard(inputs)``.

    BF16 / FP16 inputs are promoted to float32 inside the kernel (the reference promotes
    with ``.float()`` first, triton_w4a4_linear.py:599); results are identical.
    """
    if not isinstance(inputs, torch.Tensor) or not inputs.is_floating_point():
        raise TypeError("inputs must be a floating-point tensor")
    if inputs.device.type != "cuda" or inputs.ndim < 1 or inputs.numel() == 0:
        raise ValueError("inputs must be a nonempty CUDA tensor")
    if inputs.shape[-1] % 8:
        raise ValueError("activation feature dimension must be divisible by 8")
    beta_values = _beta_values(betas)
    code_width = bits_for_cardinality(q)
    beta_width = bits_for_cardinality(len(beta_values))
    if code_width not in {1, 2, 4, 8} or beta_width not in {1, 2, 4, 8}:
        raise ValueError("packed activation fields require 1, 2, 4, or 8 bits")
    if code_width != 4 or beta_width != 2:
        raise ValueError("the HIP encoder packs 4-bit codes and 2-bit beta ids (q in [9, 16], 3 or 4 betas)")
    rows = inputs.reshape(-1, inputs.shape[-1])
    if rows.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        rows = rows.float()
    rows = rows.contiguous()
    if beta_table is None:
        beta_table = torch.tensor(beta_values, device=inputs.device, dtype=torch.float32)
    decoded = torch.empty(rows.shape, dtype=torch.bfloat16, device=rows.device) if q == 14 else None
    codes, beta_ids, norms = quantize_rows_packed(rows, q=q, beta_table=beta_table, decoded=decoded,
                                                  hadamard=hadamard)
    return PreparedNQA4Activation(
        code_payload=codes, beta_payload=beta_ids, row_norms=norms, beta_table=beta_table,
        original_shape=tuple(inputs.shape), q=q, code_width=code_width, beta_width=beta_width,
        output_dtype=inputs.dtype, decoded=decoded,
    )


def fused_input_stage(inputs: torch.Tensor, *, mode: str, q: int = 14, beta_table: torch.Tensor | None = None,
                      residual: torch.Tensor | None = None, norm_weight: torch.Tensor | None = None,
                      eps: float = 0.0, gate: torch.Tensor | None = None, hadamard: bool = True,
                      encode: bool = True, want_residual: bool = False, want_staged: bool = False
                      ) -> tuple[PreparedNQA4Activation | None, torch.Tensor | None, torch.Tensor | None]:
    """Element-wise stage + rotate + encode of BF16 rows in one launch.

    mode "rmsnorm": h = inputs + residual (residual optional), y = norm_weight * rmsnorm(h);
    mode "swiglu": y = silu(gate) * inputs.  Returns (packed activation of y or None when
    `encode` is false, h when `want_residual`, y when `want_staged`), each BF16 tensor shaped
    like `inputs`.
    """
    if mode not in ("rmsnorm", "swiglu"):
        raise ValueError("mode must be 'rmsnorm' or 'swiglu'")
    device = _native.require_cuda(inputs)
    bf16 = torch.bfloat16
    if inputs.dtype != bf16 or not inputs.is_contiguous():
        raise (TypeError("the fused input stage takes BF16 tensors") if inputs.dtype != bf16
               else RuntimeError("fused input stage tensors must be contiguous"))
    for name, tensor in (("residual", residual), ("gate", gate), ("norm_weight", norm_weight)):
        if tensor is None:
            continue
        if tensor.dtype != bf16:
            raise TypeError("the fused input stage takes BF16 tensors")
        if not tensor.is_contiguous():
            raise RuntimeError("fused input stage tensors must be contiguous")
        if name != "norm_weight" and tensor.shape != inputs.shape:
            raise ValueError(f"{name} must have the shape of inputs")
    n = inputs.shape[-1]
    count = inputs.numel() // n
    if mode == "rmsnorm" and (norm_weight is None or norm_weight.numel() != n):
        raise ValueError("mode 'rmsnorm' needs a norm weight of the feature size")
    if mode == "swiglu" and gate is None:
        raise ValueError("mode 'swiglu' needs the gate rows")
    residual_out = torch.empty_like(inputs) if want_residual else None
    staged = torch.empty_like(inputs) if want_staged else None
    codes = beta_ids = norms = decoded = None
    if encode:
        if beta_table is None or q != 14 or beta_table.numel() != 4:
            raise ValueError("encoding needs q = 14 and a table of four betas")
        codes = torch.empty(count * n // 2, dtype=torch.uint8, device=device)
        beta_ids = torch.empty(count * n // 32, dtype=torch.uint8, device=device)
        norms = torch.empty(count, dtype=torch.float32, device=device)
        decoded = torch.empty((count, n), dtype=torch.bfloat16, device=device)

    def ptr(tensor):
        return None if tensor is None else tensor.data_ptr()

    _native.check(_native.library().nq_fused_input_stage(
        inputs.data_ptr(), count, n, 1 if mode == "rmsnorm" else 2, ptr(residual), ptr(residual_out),
        ptr(norm_weight), float(eps), ptr(gate), ptr(staged), q, ptr(beta_table),
        0 if beta_table is None else beta_table.numel(), int(hadamard), ptr(codes), ptr(beta_ids), ptr(norms),
        ptr(decoded), _native.stream_handle(device)))
    activation = None
    if encode:
        activation = PreparedNQA4Activation(
            code_payload=codes, beta_payload=beta_ids, row_norms=norms, beta_table=beta_table,
            original_shape=tuple(inputs.shape), q=q, code_width=4, beta_width=2,
            output_dtype=inputs.dtype, decoded=decoded)
    return activation, residual_out, staged


def quantize_weight_nqrt4(weight: torch.Tensor, *, q: int = 14, betas: Sequence[float],
                          dither_seed: int, tensor_name: str = "weight") -> PackedNestQuantTensor:
    """Quantize an (already rotated) weight [N, K] on the GPU into an NQRT v4 record with
    stateless dither: the offline step of nestquant/core/quantizer.py:214-301 followed by
    PackedNestQuantTensor.from_quantized_rows (nestquant/core/tensor_checkpoint.py:59-118)."""
    if not isinstance(weight, torch.Tensor) or not weight.is_floating_point() or weight.ndim != 2:
        raise TypeError("weight must be a floating-point matrix")
    beta_values = _beta_values(betas)
    table = torch.tensor(beta_values, device=weight.device, dtype=torch.float32)
    rows = weight.contiguous()
    dtype = rows.dtype if rows.dtype in (torch.float32, torch.bfloat16, torch.float16) else torch.float32
    codes, beta_ids, norms = quantize_rows_packed(rows.to(dtype), q=q, beta_table=table,
                                                  dither_seed=dither_seed)
    n_out, k = weight.shape
    indices = PackedNestQuantIndices((n_out, k // 8, 8), q, len(beta_values),
                                     codes.cpu().numpy().tobytes(), beta_ids.cpu().numpy().tobytes())
    return PackedNestQuantTensor(
        tensor_name=tensor_name, indices=indices, row_norms=norms.to(dtype).cpu(), betas=beta_values,
        feature_count=k, output_dtype=dtype, dither_seed=dither_seed,
        dither_algorithm=STATELESS_DITHER_ALGORITHM,
    )


def _payload_tensor(payload: bytes, device: torch.device) -> torch.Tensor:
    return torch.frombuffer(bytearray(payload), dtype=torch.uint8).to(device)


def resolve_weight(code_payload: torch.Tensor, beta_payload: torch.Tensor, *, rows: int, features: int,
                   dither_seed: int, block_offset: int = 0) -> tuple[torch.Tensor, torch.Tensor]:
    """Resolved form of an NQRT4 weight: (int32 words, int16 tails), one of each per E8 block."""
    device = _native.require_cuda(code_payload)
    blocks = rows * features // 8
    words = torch.empty(blocks, dtype=torch.int32, device=device)
    tails = torch.empty(blocks, dtype=torch.int16, device=device)
    out_of_range = torch.zeros(1, dtype=torch.int32, device=device)
    _native.check(_native.library().nq_w4a4_resolve_weight(
        code_payload.data_ptr(), beta_payload.data_ptr(), rows, features, block_offset, int(dither_seed),
        words.data_ptr(), tails.data_ptr(), out_of_range.data_ptr(), _native.stream_handle(device)))
    bad = int(out_of_range.item())
    if bad:
        raise ValueError(f"{bad} weight blocks decode outside the range of the resolved form")
    return words, tails


def prepare_fused_linear(record: Any, *, device: torch.device | str = "cuda",
                         resolve: bool = True, keep_streams: bool = False) -> PreparedNQRTLinear:
    """Copy only the packed NQRT streams and compact metadata to the target GPU, and (unless
    `resolve=False`) derive the resolved form of the weight from them.  Once a weight is resolved
    every kernel reads that form, so the device copies of the streams are dropped (6 bits per weight
    resident instead of 10.25) unless `keep_streams` asks for both."""
    for attribute in ("indices", "row_norms", "betas", "feature_count", "dither_seed",
                      "dither_algorithm", "codec_semantics"):
        if not hasattr(record, attribute):
            raise TypeError("record must be a PackedNestQuantTensor")
    target = torch.device(device)
    if target.type != "cuda" or not torch.cuda.is_available():
        raise ValueError("fused Linear preparation requires a GPU (device type 'cuda')")
    if record.dither_seed is None or record.dither_algorithm != STATELESS_DITHER_ALGORITHM:
        raise ValueError("fused Linear requires NQRT v4 stateless dither")
    if record.codec_semantics != UPSTREAM_CODEC_SEMANTICS:
        raise ValueError("fused Linear requires upstream E8 semantics")
    codes = _payload_tensor(record.indices.code_payload, target)
    beta_ids = _payload_tensor(record.indices.beta_payload, target)
    words = tails = None
    if (resolve and record.indices.q == 14 and record.indices.code_bit_width == 4
            and record.feature_count % 32 == 0 and len(record.betas) == 4):
        words, tails = resolve_weight(codes, beta_ids, rows=record.indices.shape[0],
                                      features=record.feature_count, dither_seed=record.dither_seed)
        if not keep_streams:
            codes = beta_ids = None
    return PreparedNQRTLinear(
        record=record,
        code_payload=codes,
        beta_payload=beta_ids,
        row_norms=record.row_norms.to(device=target, dtype=torch.float32),
        beta_table=torch.tensor(record.betas, device=target, dtype=torch.float32),
        resolved_words=words,
        resolved_tails=tails,
    )


# --------------------------------------------------------------------------------------
# decoders (diagnostics and container round trips)
# --------------------------------------------------------------------------------------

def dequantize_rows_packed(codes: torch.Tensor, beta_ids: torch.Tensor, norms: torch.Tensor,
                           beta_table: torch.Tensor, *, rows: int, features: int, q: int,
                           dither_seed: int | None = None, block_offset: int = 0,
                           output_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    device = _native.require_cuda(codes, beta_ids, norms, beta_table)
    out = torch.empty((rows, features), dtype=output_dtype, device=device)
    _native.check(_native.library().nq_dequantize_rows(
        codes.data_ptr(), beta_ids.data_ptr(), norms.data_ptr(), beta_table.data_ptr(), rows,
        features, q, int(dither_seed is not None), int(dither_seed or 0), block_offset,
        out.data_ptr(), _native.dtype_tag(output_dtype), _native.stream_handle(device)))
    return out


def dequantize_record(record: Any, *, device: torch.device | str = "cuda") -> torch.Tensor:
    prepared = prepare_fused_linear(record, device=device, resolve=False)
    rows = record.indices.shape[0]
    return dequantize_rows_packed(prepared.code_payload, prepared.beta_payload, prepared.row_norms,
                                  prepared.beta_table, rows=rows, features=record.feature_count,
                                  q=record.indices.q, dither_seed=record.dither_seed)


def decode_packed_a4(activation: PreparedNQA4Activation,
                     output_dtype: torch.dtype | None = None) -> torch.Tensor:
    """Decode packed NQA4 rows (diagnostic; mirrors decode_packed_a4_triton_diagnostic,
    triton_w4a4_linear.py:522-556, and decode_a4_m16 of the CUDA extension)."""
    if not isinstance(activation, PreparedNQA4Activation):
        raise TypeError("activation must be PreparedNQA4Activation")
    out = dequantize_rows_packed(
        activation.code_payload, activation.beta_payload, activation.row_norms,
        activation.beta_table, rows=activation.token_count, features=activation.feature_count,
        q=activation.q, output_dtype=output_dtype or activation.output_dtype)
    return out.reshape(*activation.original_shape)


# --------------------------------------------------------------------------------------
# predicates
# --------------------------------------------------------------------------------------

def _pointer(tensor: torch.Tensor | None) -> int | None:
    return None if tensor is None else tensor.data_ptr()


def _common_ok(activation: PreparedNQA4Activation, weight: PreparedNQRTLinear,
               feature_multiple: int, row_multiple: int) -> bool:
    record = weight.record
    streams = (weight.code_payload, weight.beta_payload)
    resolved = (weight.resolved_words, weight.resolved_tails)
    tensors = (activation.code_payload, activation.beta_payload, activation.row_norms, activation.beta_table,
               weight.row_norms, weight.beta_table, *(t for t in streams + resolved if t is not None))
    return bool(
        (all(t is not None for t in streams) or all(t is not None for t in resolved))
        and activation.feature_count == record.feature_count
        and activation.q == 14 and activation.code_width == 4 and activation.beta_width == 2
        and activation.beta_table.numel() == 4
        and record.feature_count % feature_multiple == 0
        and record.indices.shape[0] % row_multiple == 0
        and record.indices.q == 14 and record.indices.code_bit_width == 4
        and record.indices.beta_count == 4 and record.indices.beta_index_bit_width == 2
        and record.dither_seed is not None
        and record.dither_algorithm == STATELESS_DITHER_ALGORITHM
        and record.codec_semantics == UPSTREAM_CODEC_SEMANTICS
        and all(t.is_contiguous() for t in tensors)
        and all(t.device == activation.code_payload.device for t in tensors)
    )


# The HIP kernels stream 128-bit words per lane, so K must be a multiple of 32 (the
# reference's CUDA kernels accept multiples of 8 / 16); rows need no alignment.
def can_use_w4a4_gemv_m1(activation: PreparedNQA4Activation, weight: PreparedNQRTLinear) -> bool:
    return activation.token_count == 1 and _common_ok(activation, weight, 32, 1)


def can_use_w4a4_mma_small_m(activation: PreparedNQA4Activation, weight: PreparedNQRTLinear) -> bool:
    return activation.token_count in (2, 4, 8) and _common_ok(activation, weight, 32, 1)


def can_use_w4a4_mma_m16(activation: PreparedNQA4Activation, weight: PreparedNQRTLinear) -> bool:
    return activation.token_count == 16 and _common_ok(activation, weight, 128, 1)


def can_use_w4a4_mma_large_m_staged(activation: PreparedNQA4Activation,
                                    weight: PreparedNQRTLinear) -> bool:
    return activation.token_count in (32, 64, 128) and _common_ok(activation, weight, 128, 1)


def can_use_w4a4_mma_m128_staged(activation: PreparedNQA4Activation,
                                 weight: PreparedNQRTLinear) -> bool:
    return activation.token_count == 128 and can_use_w4a4_mma_large_m_staged(activation, weight)


def can_use_w4a4_mma_chunked_staged(activation: PreparedNQA4Activation,
                                    weight: PreparedNQRTLinear) -> bool:
    """Arbitrary M >= 1: the MFMA kernel pads ragged M inside the kernel."""
    return activation.token_count >= 1 and _common_ok(activation, weight, 128, 1)


# --------------------------------------------------------------------------------------
# linear kernels, M = 1..8
# --------------------------------------------------------------------------------------

# Workspaces above this size (the BF16 scratch of a decode-once prefill: 33 MB for gate_proj) are
# kept per device and stream and reused by later calls there; smaller ones are allocated
# per call from torch's caching allocator, which is what a captured graph wants.
_KEPT_WORKSPACE_BYTES = 4 << 20
_kept_workspaces: dict[tuple[int | None, int], torch.Tensor] = {}


def _workspace(device: torch.device, need: int) -> torch.Tensor:
    if need < _KEPT_WORKSPACE_BYTES or torch.cuda.is_current_stream_capturing():
        return torch.empty(need, dtype=torch.uint8, device=device)
    key = (device.index, _native.stream_handle(device))
    kept = _kept_workspaces.get(key)
    if kept is None or kept.numel() < need:
        kept = torch.empty(need, dtype=torch.uint8, device=device)
        _kept_workspaces[key] = kept
    return kept


def _gemv(activation: PreparedNQA4Activation, weight: PreparedNQRTLinear, *, split_k: int,
          output_dtype: torch.dtype, kernel: str = "gemv") -> torch.Tensor:
    lib = _native.library()
    launch = lib.nq_w4a4_gemv if kernel == "gemv" else lib.nq_w4a4_gemm
    workspace_bytes = (lib.nq_w4a4_gemv_workspace_bytes if kernel == "gemv"
                       else lib.nq_w4a4_gemm_workspace_bytes)
    device = activation.code_payload.device
    m, k, n = activation.token_count, activation.feature_count, weight.record.indices.shape[0]
    out = torch.empty((m, n), dtype=output_dtype, device=device)
    decoded = activation.decoded
    need = workspace_bytes(m, k, n, split_k, int(decoded is not None))
    workspace = _workspace(device, need) if need else None
    _native.check(launch(
        activation.code_payload.data_ptr(), activation.beta_payload.data_ptr(),
        activation.row_norms.data_ptr(), activation.beta_table.data_ptr(),
        None if decoded is None else decoded.data_ptr(), _pointer(weight.code_payload), _pointer(weight.beta_payload),
        _pointer(weight.resolved_words), _pointer(weight.resolved_tails),
        weight.row_norms.data_ptr(), weight.beta_table.data_ptr(), m, k, n, 0,
        int(weight.record.dither_seed), split_k, out.data_ptr(), _native.dtype_tag(output_dtype),
        None if workspace is None else workspace.data_ptr(), need, _native.stream_handle(device)))
    return out.reshape(*activation.original_shape[:-1], n)


def linear_packed_w4a4_gemv_grouped(activation: PreparedNQA4Activation, weights: Sequence[PreparedNQRTLinear], *,
                                    output_dtype: torch.dtype | None = None) -> list[torch.Tensor]:
    """One launch for up to four projections of the same activation of at most 8 rows (16 when K
    is a multiple of 128): q/k/v, gate/up."""
    import ctypes
    if not 1 <= len(weights) <= 4:
        raise ValueError("between one and four weights per grouped launch")
    if activation.decoded is None or any(w.resolved_words is None for w in weights):
        raise ValueError("the grouped GEMV takes a decoded activation and resolved weights")
    m, k = activation.token_count, activation.feature_count
    if not 1 <= m <= (MATRIX_CORE_GEMV_ROWS if k % 128 == 0 else 8) or any(w.record.feature_count != k for w in weights):
        raise ValueError("activation or packed weights are unsupported by the grouped W4A4 GEMV")
    dtype = output_dtype or _kernel_dtype(activation)
    device = activation.decoded.device
    count = len(weights)
    _, sizes, _, words, tails, norms, betas, widths, offsets, seeds, _ = _group_plan(weights)
    outs = [torch.empty((m, n), dtype=dtype, device=device) for n in sizes]
    _native.check(_native.library().nq_w4a4_gemv_grouped(
        activation.decoded.data_ptr(), count, words, tails, norms, betas, widths, offsets, seeds,
        (ctypes.c_void_p * count)(*[o.data_ptr() for o in outs]), m, k, _native.dtype_tag(dtype),
        _native.stream_handle(device)))
    return [o.reshape(*activation.original_shape[:-1], n) for o, n in zip(outs, sizes)]


def _kernel_dtype(activation: PreparedNQA4Activation) -> torch.dtype:
    # BF16 results are rounded once, from the FP32 accumulator, inside the kernel; any
    # other output dtype goes through FP32 exactly like the reference's `.to(dtype)`.
    return torch.bfloat16 if activation.output_dtype == torch.bfloat16 else torch.float32


def linear_packed_w4a4_gemv_m1(activation: PreparedNQA4Activation,
                               weight: PreparedNQRTLinear) -> torch.Tensor:
    """Packed-word direct W4A4 GEMV for one token."""
    if not can_use_w4a4_gemv_m1(activation, weight):
        raise ValueError("activation or packed weight is unsupported by W4A4 M1")
    return _gemv(activation, weight, split_k=0,
                 output_dtype=_kernel_dtype(activation)).to(activation.output_dtype)


def linear_packed_w4a4_gemv_m1_fp32_probe(activation: PreparedNQA4Activation,
                                          weight: PreparedNQRTLinear) -> torch.Tensor:
    """The M1 accumulator before output-dtype rounding."""
    if not can_use_w4a4_gemv_m1(activation, weight):
        raise ValueError("activation or packed weight is unsupported by W4A4 M1")
    return _gemv(activation, weight, split_k=0, output_dtype=torch.float32)


def linear_packed_w4a4_gemv_m1_splitk_probe(activation: PreparedNQA4Activation,
                                            weight: PreparedNQRTLinear, *,
                                            split_k: int) -> torch.Tensor:
    """Deterministic long-K M1 split-K: slices are reduced in ascending order."""
    if not can_use_w4a4_gemv_m1(activation, weight):
        raise ValueError("activation or packed weight is unsupported by W4A4 M1")
    if split_k not in (2, 4, 8):
        raise ValueError("split_k must be 2, 4, or 8")
    return _gemv(activation, weight, split_k=split_k,
                 output_dtype=_kernel_dtype(activation)).to(activation.output_dtype)


def linear_packed_w4a4_gemv_m1_splitk_fp32_probe(activation: PreparedNQA4Activation,
                                                 weight: PreparedNQRTLinear, *,
                                                 split_k: int) -> torch.Tensor:
    if not can_use_w4a4_gemv_m1(activation, weight):
        raise ValueError("activation or packed weight is unsupported by W4A4 M1")
    if split_k not in (2, 4, 8):
        raise ValueError("split_k must be 2, 4, or 8")
    return _gemv(activation, weight, split_k=split_k, output_dtype=torch.float32)


def linear_packed_w4a4_mma_small_m(activation: PreparedNQA4Activation,
                                   weight: PreparedNQRTLinear) -> torch.Tensor:
    """M in {2, 4, 8}: each weight block is decoded once and reused by every token."""
    if not can_use_w4a4_mma_small_m(activation, weight):
        raise ValueError("activation or packed weight is unsupported by small-M probe")
    return _gemv(activation, weight, split_k=0,
                 output_dtype=_kernel_dtype(activation)).to(activation.output_dtype)


def linear_packed_w4a4_mma_small_m_splitk_probe(activation: PreparedNQA4Activation,
                                                weight: PreparedNQRTLinear, *,
                                                split_k: int) -> torch.Tensor:
    if not can_use_w4a4_mma_small_m(activation, weight):
        raise ValueError("activation or packed weight is unsupported by small-M")
    if split_k not in (2, 4, 8):
        raise ValueError("split_k must be 2, 4, or 8")
    return _gemv(activation, weight, split_k=split_k,
                 output_dtype=_kernel_dtype(activation)).to(activation.output_dtype)


# --------------------------------------------------------------------------------------
# linear kernels, prefill (matrix cores)
# --------------------------------------------------------------------------------------

# From this many rows on (BF16 output, automatic split) nq_w4a4_gemm decodes the weight once into a
# BF16 scratch inside its workspace and multiplies with the dense matrix-core GEMM of the library
# (nq_bf16_gemm); below, the fused kernel decodes inside the multiply.  Measured on MI355X at the 1B
# shapes: gate + up 50 us at 256 rows on the fused kernel, 101 us at 257 (a second token tile per
# wavefront), 68 us on this route.
DECODE_ONCE_ROWS = 257
# up to this many rows a linear over resolved weights (K a multiple of 128) takes the decode GEMV,
# which from two rows on multiplies on the matrix cores
MATRIX_CORE_GEMV_ROWS = 16
BF16_ROWS_LINEAR_MAX_ROWS = 16
BF16_ROWS_LINEAR_K = (2048, 4096, 8192)


def decode_weight_bf16(weight: PreparedNQRTLinear, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """The BF16 weight [N, K] the packed linear kernels multiply by (transient scratch); into `out`
    (contiguous BF16 [N, K] on the weight's device) when given."""
    device = weight.row_norms.device
    n, k = weight.record.indices.shape[0], weight.record.feature_count
    if out is None:
        out = torch.empty((n, k), dtype=torch.bfloat16, device=device)
    elif tuple(out.shape) != (n, k) or out.dtype != torch.bfloat16 or not out.is_contiguous() or out.device != device:
        raise ValueError("out must be a contiguous BF16 [N, K] tensor on the weight's device")
    _native.check(_native.library().nq_w4a4_decode_weight(
        _pointer(weight.code_payload), _pointer(weight.beta_payload), _pointer(weight.resolved_words),
        _pointer(weight.resolved_tails),
        weight.row_norms.data_ptr(), weight.beta_table.data_ptr(), n, k, 0, int(weight.record.dither_seed),
        out.data_ptr(), _native.stream_handle(device)))
    return out


def can_use_bf16_rows_linear(rows: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether `bf16_rows_linear` takes this activation and weight."""
    return (rows.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and rows.device.type == "cuda"
            and weight.device == rows.device and rows.ndim == 2 and weight.ndim == 2
            and 1 <= rows.shape[0] <= BF16_ROWS_LINEAR_MAX_ROWS and rows.shape[1] == weight.shape[1]
            and weight.shape[1] in BF16_ROWS_LINEAR_K and rows.is_contiguous() and weight.is_contiguous()
            and rows.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def bf16_rows_linear(rows: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """`rows @ weight.T` for at most 16 BF16 rows against a BF16 [N, K] weight (K 2048, 4096 or
    8192), FP32 accumulation, BF16 out: the LM head of a decode step
    (nestquant/runtime/nqkv_batched_runner.py:162-169) as one stream over the weight."""
    return bf16_rows_linear_grouped(rows, weight, [weight.shape[0]])[0]


def bf16_rows_linear_grouped(rows: torch.Tensor, weight: torch.Tensor, sizes: Sequence[int]) -> list[torch.Tensor]:
    """`bf16_rows_linear` against a weight whose N rows are the rows of up to three projections of
    the same activation, one after the other (`sizes` rows each): one launch, one dense BF16
    [rows, size] output per projection."""
    if not can_use_bf16_rows_linear(rows, weight):
        raise ValueError("bf16_rows_linear takes contiguous BF16 [rows <= 16, K] and [N, K] on one GPU, "
                         "K 2048, 4096 or 8192")
    sizes = [int(size) for size in sizes]
    if not 1 <= len(sizes) <= 3 or min(sizes) < 1 or sum(sizes) != weight.shape[0]:
        raise ValueError("between one and three positive sizes that add up to the weight's rows")
    device = _native.require_cuda(rows)
    outs = [torch.empty((rows.shape[0], size), dtype=torch.bfloat16, device=device) for size in sizes]
    group_n = (ctypes.c_int64 * len(sizes))(*sizes)
    pointers = (ctypes.c_void_p * len(sizes))(*[out.data_ptr() for out in outs])
    _native.check(_native.library().nq_bf16_rows_linear_grouped(
        rows.data_ptr(), weight.data_ptr(), rows.shape[0], rows.shape[1], len(sizes), group_n, pointers,
        _native.stream_handle(device)))
    return outs


def _gemm(activation: PreparedNQA4Activation, weight: PreparedNQRTLinear, *,
          output_dtype: torch.dtype | None = None, split_k: int = 0) -> torch.Tensor:
    dtype = _kernel_dtype(activation) if output_dtype is None else output_dtype
    if (split_k == 0 and activation.token_count <= MATRIX_CORE_GEMV_ROWS and weight.resolved_words is not None
            and activation.feature_count % 128 == 0):
        # up to sixteen rows the decode-in-register kernel feeds the matrix cores directly
        return _gemv(activation, weight, split_k=0, output_dtype=dtype)
    return _gemv(activation, weight, split_k=split_k, output_dtype=dtype, kernel="gemm")


def bf16_gemm(rows: torch.Tensor, weight: torch.Tensor, *, tile: int = -1, split_k: int = 0) -> torch.Tensor:
    """`rows @ weight.T` for BF16 [M, K] and [N, K] (K a multiple of 128) on the library's dense
    matrix-core GEMM, FP32 accumulation, BF16 out.  `tile` forces a workgroup tile and `split_k` a K
    split (measurements); by default the library splits K when the product has few tiles."""
    device = _native.require_cuda(rows, weight)
    if rows.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or rows.ndim != 2 or weight.ndim != 2:
        raise TypeError("bf16_gemm takes two BF16 matrices")
    if rows.shape[1] != weight.shape[1]:
        raise ValueError("operands disagree on K")
    m, n = rows.shape[0], weight.shape[0]
    out = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    need = 8 * m * n * 4 if m * n <= (1 << 22) else 0               # room for the widest split of a small product
    workspace = _workspace(device, need) if need else None
    _native.check(_native.library().nq_bf16_gemm(rows.data_ptr(), weight.data_ptr(), m, n, rows.shape[1], out.data_ptr(),
                                                 tile, split_k, None if workspace is None else workspace.data_ptr(), need,
                                                 _native.stream_handle(device)))
    return out


FUSED_GROUP_MAX_ROWS = 512                  # one chunk of the fused kernel

# What a grouped launch passes for its weights never changes while the weights live: the pointer,
# size, offset and seed arrays are built once per group (keyed by the weights' identities, dropped
# with the first weight that is collected).
_group_plans: dict[tuple[int, ...], tuple] = {}


def _group_plan(weights: Sequence[PreparedNQRTLinear]) -> tuple:
    """(weak references, sizes, their sum, words, tails, norms, betas, sizes as int, zero offsets,
    seeds, sizes as int64) of the resolved weights of one grouped launch."""
    key = tuple(id(w) for w in weights)
    plan = _group_plans.get(key)
    if plan is not None and all(ref() is w for ref, w in zip(plan[0], weights)):
        return plan
    count = len(weights)
    array = ctypes.c_void_p * count
    sizes = [int(w.record.indices.shape[0]) for w in weights]
    forget = lambda _, key=key: _group_plans.pop(key, None)
    plan = (tuple(weakref.ref(w, forget) for w in weights), sizes, sum(sizes),
            array(*[w.resolved_words.data_ptr() for w in weights]),
            array(*[w.resolved_tails.data_ptr() for w in weights]),
            array(*[w.row_norms.data_ptr() for w in weights]),
            array(*[w.beta_table.data_ptr() for w in weights]),
            (ctypes.c_int * count)(*sizes), (ctypes.c_int64 * count)(*([0] * count)),
            (ctypes.c_int64 * count)(*[int(w.record.dither_seed) for w in weights]),
            (ctypes.c_int64 * count)(*sizes))
    _group_plans[key] = plan
    return plan


class StageLinearSync:
    """The hand-over state of `fused_stage_linear` launches on one stream: sets of flag words (one
    set per launch), the status word a consumer sets when its bounded wait runs out (pinned host
    memory: the host looks at it without a synchronisation), and the number of polls of that wait.

    Two ways to hand out the sets.  A caller that issues a fixed sequence of launches again and
    again (a decode step, also as a captured graph) calls `begin_step()` first: one fill clears
    every set, and the launches of the step take sets 0, 1, ... .  Without `begin_step` the sets
    form a ring in which every launch clears the set of the launch before it."""

    def __init__(self, device: torch.device, *, sets: int = 128, spin_limit: int = 400_000) -> None:
        if sets < 2:
            raise ValueError("at least two sets of flag words")
        # words per set: what the largest launch asks for (the library keeps several copies of a launch's flags)
        self.set_words = int(_native.library().nq_fused_stage_linear_flag_words(16, 2048))
        self.flags = torch.zeros((sets, self.set_words), dtype=torch.int32, device=device)
        self.status = torch.zeros(1, dtype=torch.int32).pin_memory()
        self.spin_limit = int(spin_limit)
        self._next = 0
        self._previous: tuple[int, int] | None = None       # (set, words) of the launch before, ring form
        self._in_step = False

    def begin_step(self) -> None:
        """Clear every set with one fill (capturable) and hand the sets out from the first again."""
        self.flags.zero_()
        self._next, self._previous, self._in_step = 0, None, True

    def take(self, words: int) -> tuple[int, int | None, int]:
        """(pointer to this launch's flag words, pointer to the words this launch clears or None, their count)."""
        if not 1 <= words <= self.set_words:
            raise ValueError(f"a launch takes between 1 and {self.set_words} flag words")
        current = self._next
        if self._in_step:
            if current >= self.flags.shape[0]:
                raise RuntimeError("more launches in a step than sets of flag words")
            self._next = current + 1
            return self.flags[current].data_ptr(), None, 0
        self._next = (current + 1) % self.flags.shape[0]
        previous = self._previous
        self._previous = (current, words)
        here = self.flags[current].data_ptr()
        if previous is None:
            return here, None, 0
        return here, self.flags[previous[0]].data_ptr(), previous[1]

    @property
    def timed_out(self) -> bool:
        return bool(self.status[0].item())

    def reset(self) -> None:
        """After a time-out: every flag word and the status back to zero (the stream must be idle)."""
        self.flags.zero_()
        self.status.zero_()
        self._next, self._previous, self._in_step = 0, None, False


def can_use_fused_stage_linear(rows: int, k: int, weights: Sequence[PreparedNQRTLinear]) -> bool:
    """Whether `fused_stage_linear` takes this decode-step pair: up to 16 rows of 2048 or
    8192 values, one to four resolved weights of that K."""
    return k in (2048, 8192) and 1 <= rows <= 16 and 1 <= len(weights) <= 4 and all(
        w.resolved_words is not None and w.record.feature_count == k for w in weights)


def fused_stage_linear(inputs: torch.Tensor | None, weights: Sequence[PreparedNQRTLinear], sync: StageLinearSync, *,
                       mode: str, beta_table: torch.Tensor, residual: torch.Tensor | None = None,
                       norm_weight: torch.Tensor | None = None, eps: float = 0.0, gate: torch.Tensor | None = None,
                       attention_workspace=None, want_residual: bool = False, want_staged: bool = False,
                       output_dtype: torch.dtype = torch.bfloat16
                       ) -> tuple[list[torch.Tensor], PreparedNQA4Activation, torch.Tensor | None, torch.Tensor | None]:
    """`fused_input_stage` (mode "rmsnorm" / "swiglu") or `attention_output_stage` (mode "attention", the
    rows then come from `attention_workspace`, a BatchedNQKVAttentionWorkspace whose first stage has run)
    with the Hadamard rotation, or the encoder alone on the rows themselves (mode "rows": rotated first, as
    `quantize_activation_cuda(..., hadamard=True)`; mode "rotated_rows": as they are), followed by `linear_packed_w4a4_gemv_grouped` of `weights` on the encoded
    rows, as one launch whose linear workgroups decode their weights while the encoder runs.  Returns
    (outputs, packed activation, residual sum when `want_residual`, staged rows when `want_staged`): the
    same bits as the two calls.  `sync` orders the launch among its neighbours on the stream."""
    if mode not in ("rmsnorm", "swiglu", "attention", "rows", "rotated_rows"):
        raise ValueError("mode must be 'rmsnorm', 'swiglu', 'attention', 'rows' or 'rotated_rows'")
    bf16 = torch.bfloat16
    if mode == "attention":
        if attention_workspace is None:
            raise ValueError("mode 'attention' needs the attention workspace")
        device = attention_workspace.buffer.device
        rows, n = attention_workspace.batch_size, attention_workspace.query_heads * attention_workspace.head_dim
        shape = (rows, n)
    else:
        device = _native.require_cuda(inputs)
        if inputs.dtype != bf16:
            raise TypeError("the fused input stage takes BF16 tensors")
        if not inputs.is_contiguous():
            raise RuntimeError("fused input stage tensors must be contiguous")
        n = inputs.shape[-1]
        rows = inputs.numel() // n
        shape = tuple(inputs.shape)
        for name, tensor in (("residual", residual), ("gate", gate), ("norm_weight", norm_weight)):
            if tensor is None:
                continue
            if tensor.dtype != bf16:
                raise TypeError("the fused input stage takes BF16 tensors")
            if not tensor.is_contiguous():
                raise RuntimeError("fused input stage tensors must be contiguous")
            if name != "norm_weight" and tensor.shape != inputs.shape:
                raise ValueError(f"{name} must have the shape of inputs")
        if mode == "rmsnorm" and (norm_weight is None or norm_weight.numel() != n):
            raise ValueError("mode 'rmsnorm' needs a norm weight of the feature size")
        if mode == "swiglu" and gate is None:
            raise ValueError("mode 'swiglu' needs the gate rows")
        if mode in ("rows", "rotated_rows") and (want_staged or want_residual or residual is not None or gate is not None):
            raise ValueError("modes 'rows' and 'rotated_rows' have no staged rows, residual or gate")
    if not can_use_fused_stage_linear(rows, n, weights):
        raise ValueError("rows, K or weights are outside what the fused stage + linear launch takes")
    if beta_table is None or beta_table.numel() != 4:
        raise ValueError("encoding needs a table of four betas")
    if output_dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("outputs are BF16 or float32")
    lib = _native.library()
    residual_out = torch.empty(shape, dtype=bf16, device=device) if (want_residual and mode == "rmsnorm") else None
    staged = torch.empty(shape, dtype=bf16, device=device) if want_staged else None
    codes = torch.empty(rows * n // 2, dtype=torch.uint8, device=device)
    beta_ids = torch.empty(rows * n // 32, dtype=torch.uint8, device=device)
    norms = torch.empty(rows, dtype=torch.float32, device=device)
    decoded = torch.empty((rows, n), dtype=bf16, device=device)
    count = len(weights)
    _, sizes, _, words, tails, w_norms, w_betas, widths, offsets, seeds, _ = _group_plan(weights)
    outs = [torch.empty((rows, size), dtype=output_dtype, device=device) for size in sizes]
    flags, previous, previous_words = sync.take(lib.nq_fused_stage_linear_flag_words(rows, n))

    def ptr(tensor):
        return None if tensor is None else tensor.data_ptr()

    parts = 0 if mode != "attention" else lib.nq_nqkv_attention_parts(rows, attention_workspace.max_pages)
    _native.check(lib.nq_fused_stage_linear(
        ptr(inputs) if mode != "attention" else None, rows, n,
        {"rows": 0, "rmsnorm": 1, "swiglu": 2, "attention": 3, "rotated_rows": 4}[mode],
        ptr(residual), ptr(residual_out), ptr(norm_weight), float(eps), ptr(gate),
        attention_workspace.buffer.data_ptr() if mode == "attention" else None,
        attention_workspace.query_heads if mode == "attention" else 0, parts, ptr(staged), beta_table.data_ptr(), 4,
        codes.data_ptr(), beta_ids.data_ptr(), norms.data_ptr(), decoded.data_ptr(), count, words, tails, w_norms, w_betas,
        widths, offsets, seeds, (ctypes.c_void_p * count)(*[o.data_ptr() for o in outs]), _native.dtype_tag(output_dtype),
        flags, previous, previous_words, sync.status.data_ptr(), sync.spin_limit, _native.stream_handle(device)))
    activation = PreparedNQA4Activation(
        code_payload=codes, beta_payload=beta_ids, row_norms=norms, beta_table=beta_table, original_shape=shape, q=14,
        code_width=4, beta_width=2, output_dtype=bf16, decoded=decoded)
    return [o.reshape(*shape[:-1], size) for o, size in zip(outs, sizes)], activation, residual_out, staged


def _fused_group(activation: PreparedNQA4Activation, weights: Sequence[PreparedNQRTLinear]) -> bool:
    """A group the fused kernel takes in one launch: a prefill below the decode-once size."""
    return (MATRIX_CORE_GEMV_ROWS < activation.token_count < DECODE_ONCE_ROWS and 2 <= len(weights) <= 4
            and all(w.resolved_words is not None and w.record.indices.shape[0] % 32 == 0 for w in weights))


def can_use_w4a4_gemm_grouped(activation: PreparedNQA4Activation, weights: Sequence[PreparedNQRTLinear]) -> bool:
    """Whether `linear_packed_w4a4_gemm_grouped` takes these projections of one decoded activation:
    a long prefill (the decode-once route: two or three weights, every N a multiple of 256), or a
    shorter one of more than 16 rows (the fused kernel: up to four resolved weights, every N a
    multiple of 32)."""
    k = activation.feature_count
    if k % 128 != 0 or activation.decoded is None or any(w.record.feature_count != k for w in weights):
        return False
    if _fused_group(activation, weights):
        return True
    return (2 <= len(weights) <= 3 and activation.token_count >= DECODE_ONCE_ROWS
            and all(w.record.indices.shape[0] % 256 == 0 for w in weights))


def linear_packed_w4a4_gemm_grouped(activation: PreparedNQA4Activation, weights: Sequence[PreparedNQRTLinear], *,
                                    checked: bool = False) -> list[torch.Tensor]:
    """The linears of the weights that share one activation (q, k and v; gate and up) in a prefill,
    as one product.  From 257 rows on every weight is decoded once into its rows of one BF16 scratch
    and one dense matrix-core GEMM over the stacked rows stores each projection's columns to a BF16
    [M, N_i] output of its own; below, one launch of the fused kernel walks the channels of all the
    weights.  Same values as one `linear_packed_w4a4_mma_chunked_staged` per weight.  `checked`:
    the caller has just asked `can_use_w4a4_gemm_grouped`."""
    if not checked and not can_use_w4a4_gemm_grouped(activation, weights):
        raise ValueError("grouped prefill linears take the weights of one decoded activation, K a multiple of 128: "
                         f"2 or 3 with every N a multiple of 256 from {DECODE_ONCE_ROWS} rows on, up to 4 resolved "
                         f"ones with every N a multiple of 32 between {MATRIX_CORE_GEMV_ROWS + 1} rows and that")
    rows = activation.decoded.reshape(activation.token_count, activation.feature_count)
    device = _native.require_cuda(rows)
    m, k = rows.shape
    count = len(weights)
    lib = _native.library()
    if _fused_group(activation, weights):
        _, sizes, total, words, tails, norms, betas, widths, offsets, seeds, _ = _group_plan(weights)
        outs = [torch.empty((m, size), dtype=torch.bfloat16, device=device) for size in sizes]
        pointers = (ctypes.c_void_p * count)(*[out.data_ptr() for out in outs])
        need = lib.nq_w4a4_gemm_grouped_workspace_bytes(m, k, total)
        workspace = _workspace(device, need) if need else None
        _native.check(lib.nq_w4a4_gemm_grouped(
            rows.data_ptr(), count, words, tails, norms, betas, widths, offsets, seeds, pointers, m, k,
            None if workspace is None else workspace.data_ptr(), need, _native.stream_handle(device)))
    else:
        sizes = [int(w.record.indices.shape[0]) for w in weights]
        outs = [torch.empty((m, size), dtype=torch.bfloat16, device=device) for size in sizes]
        pointers = (ctypes.c_void_p * count)(*[out.data_ptr() for out in outs])
        stacked = _workspace(device, sum(sizes) * k * 2)[: sum(sizes) * k * 2].view(torch.bfloat16).view(sum(sizes), k)
        first = 0
        for weight, size in zip(weights, sizes):
            decode_weight_bf16(weight, out=stacked[first:first + size])
            first += size
        widths = (ctypes.c_int64 * count)(*sizes)
        _native.check(lib.nq_bf16_gemm_split(rows.data_ptr(), stacked.data_ptr(), m, k, pointers, widths, count, -1,
                                             _native.stream_handle(device)))
    return [out.reshape(*activation.original_shape[:-1], size) for out, size in zip(outs, sizes)]


def linear_packed_w4a4_mma_m16(activation: PreparedNQA4Activation,
                               weight: PreparedNQRTLinear) -> torch.Tensor:
    if not can_use_w4a4_mma_m16(activation, weight):
        raise ValueError("activation or packed weight is unsupported by W4A4 M16")
    return _gemm(activation, weight).to(activation.output_dtype)


def linear_packed_w4a4_mma_large_m_staged(activation: PreparedNQA4Activation,
                                          weight: PreparedNQRTLinear) -> torch.Tensor:
    """M in {32, 64, 128}: decoded weight fragments staged once per workgroup in LDS."""
    if not can_use_w4a4_mma_large_m_staged(activation, weight):
        raise ValueError("activation or packed weight is unsupported by staged large-M")
    return _gemm(activation, weight).to(activation.output_dtype)


def linear_packed_w4a4_mma_m128_staged(activation: PreparedNQA4Activation,
                                       weight: PreparedNQRTLinear) -> torch.Tensor:
    if not can_use_w4a4_mma_m128_staged(activation, weight):
        raise ValueError("activation or packed weight is unsupported by staged M128")
    return _gemm(activation, weight).to(activation.output_dtype)


def linear_packed_w4a4_mma_chunked_staged(activation: PreparedNQA4Activation,
                                          weight: PreparedNQRTLinear) -> torch.Tensor:
    """Arbitrary M.  The reference covers M with 128-row chunks plus a tail padded to the
    next supported size (cuda_w4a4_mma.py:450-474); here one launch handles up to 512 rows
    and pads the ragged tail to a multiple of 32 with zero rows inside the kernel, so every
    weight block is decoded once per 512 rows instead of once per 128."""
    if not can_use_w4a4_mma_chunked_staged(activation, weight):
        raise ValueError("activation or packed weight is unsupported by chunked staged")
    return _gemm(activation, weight).to(activation.output_dtype)


linear_packed_w4a4_mma_chunked_staged_probe = linear_packed_w4a4_mma_chunked_staged


def slice_pad_packed_activation_rows(activation: PreparedNQA4Activation, start: int, row_count: int,
                                     padded_row_count: int) -> PreparedNQA4Activation:
    """Slice row-aligned packed A4 payloads and append zero-norm padding rows
    (nestquant/runtime/cuda_w4a4_mma.py:393-447).  Padding rows carry zero codes and a zero
    norm, so they decode to exact zeros."""
    if not 0 <= start < activation.token_count:
        raise ValueError("packed activation slice start is out of range")
    if row_count < 1 or start + row_count > activation.token_count:
        raise ValueError("packed activation slice row count is out of range")
    if padded_row_count < row_count:
        raise ValueError("padded row count must cover the activation slice")
    k = activation.feature_count
    pad = padded_row_count - row_count

    def cut(payload: torch.Tensor, per_row: int) -> torch.Tensor:
        piece = payload[start * per_row:(start + row_count) * per_row]
        if not pad:
            return piece.contiguous()
        return torch.cat((piece, torch.zeros(pad * per_row, dtype=payload.dtype, device=payload.device)))

    decoded = None
    if activation.decoded is not None:
        decoded = cut(activation.decoded.reshape(-1), k).reshape(padded_row_count, k)
    return PreparedNQA4Activation(
        code_payload=cut(activation.code_payload, k * activation.code_width // 8),
        beta_payload=cut(activation.beta_payload, (k // 8) * activation.beta_width // 8),
        row_norms=cut(activation.row_norms, 1), beta_table=activation.beta_table,
        original_shape=(padded_row_count, k), q=activation.q, code_width=activation.code_width,
        beta_width=activation.beta_width, output_dtype=activation.output_dtype, decoded=decoded,
    )
