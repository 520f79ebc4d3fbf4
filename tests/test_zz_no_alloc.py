"""nq_w4a4_gemv_static (the entry point that allocates nothing) against nq_w4a4_gemv, through
the C ABI: same kernels, so the outputs must agree bit for bit.  Two calls in a row share the
library's built-in scratch buffer; the second is smaller, so whatever the first left behind
must not leak into it."""

import numpy as np
import pytest
import torch

from conftest import ACTIVATION_BETAS, Q, WEIGHT_BETAS
from gpu_util import bits, oracle_weight, relative_error, student_t_rows

pytestmark = pytest.mark.gpu


def _case(oracle, rt, m, k, n_out, seed):
    from test_gpu_gemv import _record, _references
    _, wc, wb, wn = oracle_weight(oracle, n_out, k, seed=3000 + k + n_out, dither_seed=seed)
    weight = rt.prepare_fused_linear(_record(rt, wc, wb, wn, k, seed), device="cuda", keep_streams=True)
    x = torch.from_numpy(oracle.hadamard(student_t_rows(m, k, seed=4001 + m).numpy())).to(torch.bfloat16).cuda()
    activation = rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS)
    ref32, _ = _references(oracle, activation, rt, wc, wb, wn, seed)
    return activation, weight, ref32, seed


def _call(entry, activation, weight, seed, split_k, with_decoded, resolved, workspace):
    from nestquant_aiinfra_amd import _native
    lib = _native.library()
    m, k, n = activation.token_count, activation.feature_count, weight.record.indices.shape[0]
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    decoded = activation.decoded if with_decoded else None
    arguments = [
        activation.code_payload.data_ptr(), activation.beta_payload.data_ptr(), activation.row_norms.data_ptr(),
        activation.beta_table.data_ptr(), None if decoded is None else decoded.data_ptr(),
        weight.code_payload.data_ptr(), weight.beta_payload.data_ptr(),
        weight.resolved_words.data_ptr() if resolved else None, weight.resolved_tails.data_ptr() if resolved else None,
        weight.row_norms.data_ptr(), weight.beta_table.data_ptr(), m, k, n, 0, seed, split_k, out.data_ptr(),
        _native.NQ_F32]
    stream = _native.stream_handle(out.device)
    if entry == "static":
        _native.check(lib.nq_w4a4_gemv_static(*arguments, stream))
    else:
        need = lib.nq_w4a4_gemv_workspace_bytes(m, k, n, split_k, int(decoded is not None))
        assert workspace.numel() >= need
        _native.check(lib.nq_w4a4_gemv(*arguments, workspace.data_ptr() if need else None, need, stream))
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("resolved", [True, False])
def test_static_scratch_gemv_equals_the_workspace_gemv(oracle, resolved):
    from nestquant_aiinfra_amd.runtime import w4a4_linear as rt
    workspace = torch.empty(8 << 20, dtype=torch.uint8, device="cuda")
    # first call: eight rows, packed activation decoded into the scratch, K split four ways
    big = _case(oracle, rt, 8, 8192, 256, 20261201)
    # second call: smaller in every dimension, explicit two-way split
    small = _case(oracle, rt, 2, 2048, 136, 20261202)
    for (activation, weight, ref32, seed), split_k in ((big, 0), (small, 2), (big, 8), (small, 1)):
        for with_decoded in (False, True):
            workspace.fill_(0xA5)
            expected = _call("workspace", activation, weight, seed, split_k, with_decoded, resolved, workspace)
            actual = _call("static", activation, weight, seed, split_k, with_decoded, resolved, workspace)
            assert torch.equal(actual, expected)
            assert relative_error(bits(actual), ref32) <= 1e-2


def test_static_scratch_gemv_allocates_no_device_memory(oracle):
    """The property the entry point exists for: once the library is warm, a call changes neither
    the device's free memory nor what the framework's allocator holds."""
    from nestquant_aiinfra_amd import _native
    from nestquant_aiinfra_amd.runtime import w4a4_linear as rt
    lib = _native.library()
    _native.check(lib.nq_w4a4_gemv_static_init())
    activation, weight, ref32, seed = _case(oracle, rt, 8, 8192, 256, 20261203)
    m, k, n = activation.token_count, activation.feature_count, weight.record.indices.shape[0]
    out = torch.empty((m, n), dtype=torch.float32, device="cuda")
    arguments = [
        activation.code_payload.data_ptr(), activation.beta_payload.data_ptr(), activation.row_norms.data_ptr(),
        activation.beta_table.data_ptr(), None, None, None,
        weight.resolved_words.data_ptr(), weight.resolved_tails.data_ptr(), weight.row_norms.data_ptr(),
        weight.beta_table.data_ptr(), m, k, n, 0, seed, 4, out.data_ptr(), _native.NQ_F32,
        _native.stream_handle(out.device)]
    _native.check(lib.nq_w4a4_gemv_static(*arguments))                   # warm: code objects loaded
    torch.cuda.synchronize()
    free_before, reserved_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    for _ in range(3):
        _native.check(lib.nq_w4a4_gemv_static(*arguments))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == reserved_before
    assert relative_error(bits(out), ref32) <= 1e-2


def test_static_scratch_gemv_rejects_what_does_not_fit():
    from nestquant_aiinfra_amd import _native
    lib = _native.library()
    # 8 rows x 8 slices x 32768 channels of float32 partials = 8 MiB > the 4 MiB buffer
    status = lib.nq_w4a4_gemv_static(*([None] * 11), 8, 8192, 32768, 0, 1, 8, None, 0, None)
    assert status == _native.NQ_ERR_WORKSPACE and b"built-in buffer holds" in lib.nq_last_error()
    with pytest.raises(RuntimeError, match="caller-owned workspace"):
        _native.check(status)
