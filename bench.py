"""Benchmark of the packed W4A4 decode path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the configuration the headline metric is quoted on): single W4A4 decode linear
at Llama-3.2-1B projection shapes, q_proj (K = 2048, N = 2048) and down_proj (K = 8192,
N = 2048), each at M = 1 and M = 8.  Weights are NQRT4 records quantised on the GPU from
Hadamard-rotated N(0, 0.02) matrices; activations are BF16 Student-t(4) rows, Hadamard
rotated.  One step = for each of the four cases: NQA4-encode the activation on the GPU,
then run the packed linear.  Inputs and weights are resident in HBM before the timed
region; weights rotate over distinct copies (> 600 MB in total) so that no step finds its
weights in the 256 MB last-level cache.  Each step is a captured HIP graph.

`value` = algorithmic bytes of the four linears per step / wall time per step (GB/s):
N*K/2 + N*K/32 + 4N + 16 (NQRT4) + M*(K/2 + K/32 + 4) + 16 (NQA4) + 2*M*N (BF16 out).
`roofline` covers the dominant kernel, timed alone with events on its own stream;
`cpu_baseline` is the CPU oracle (a C restatement of the reference's CPU codec +
decoded matmul) on a bounded sample of the same workload.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

Q = 14
ACTIVATION_BETAS = tuple(v / 14 for v in (3.47, 4.74, 6.90, 18.11))
WEIGHT_BETAS = tuple(v / 14 for v in (4.0, 5.5, 7.0, 18.0))
HBM_PEAK_GBPS = 8000.0
SHAPES = (("q_proj", 2048, 2048, 1001, 20261101), ("down_proj", 8192, 2048, 1002, 20261102))
TOKEN_COUNTS = (1, 8)
MIN_ROTATION_BYTES = 600 * 1024 * 1024


def linear_bytes(m: int, k: int, n: int) -> int:
    return n * k // 2 + n * k // 32 + 4 * n + 16 + m * (k // 2 + k // 32 + 4) + 16 + 2 * m * n


# HBM bytes per launch of the linear kernel come from counters (FETCH_SIZE + WRITE_SIZE of rocprofv3
# --pmc, scaled by what the same counters read for a 256 MiB copy), which cannot be read from inside
# this process: the profile summary below holds them in its "traffic bytes" column, together with a
# fingerprint of the kernel sources it was taken on.  A summary taken on other sources is stale and
# reads as None.
TRAFFIC_PROFILE = ROOT / "profiles" / "w4a4_gemv_decode_rocprofv3.md"
KERNEL_SOURCES = ("nq_gemv.hip", "nq_e8.hip.h", "nq_linear_common.hip.h")


def kernel_source_fingerprint() -> str:
    import hashlib
    digest = hashlib.sha256()
    for name in KERNEL_SOURCES:
        digest.update((ROOT / "nestquant_aiinfra_amd" / "csrc" / name).read_bytes())
    return digest.hexdigest()[:16]


def measured_traffic_bytes(case_name: str):
    """`traffic bytes` of e.g. "down_proj_m1" from the profile summary, or None when the summary is
    missing, does not list the case, or was taken on kernel sources other than the current ones."""
    try:
        lines = TRAFFIC_PROFILE.read_text().splitlines()
    except OSError:
        return None
    if not any(line.startswith("Kernel source fingerprint:") and kernel_source_fingerprint() in line for line in lines):
        return None
    name, rows = case_name.rsplit("_m", 1)
    label = f"{name} M={rows} |"
    for line in lines:
        cells = [cell.strip() for cell in line.strip().strip("|").split("|")]
        if label in line and len(cells) == 8 and cells[-1].isdigit():
            return int(cells[-1])
    return None


# the kernel each case launches (one row: vector units; eight rows: matrix cores, two K ranges per tile)
CASE_KERNEL = {"q_proj_m1": "w4a4_gemv_kernel<1, 2, true>", "down_proj_m1": "w4a4_gemv_kernel<1, 2, true>",
               "q_proj_m8": "w4a4_gemv_mfma_kernel<2>", "down_proj_m8": "w4a4_gemv_mfma_kernel<2>"}


def parse_args() -> argparse.Namespace:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=200)
    parser.add_argument("--warmup", type=int, default=20)
    parser.add_argument("--skip-cpu-baseline", action="store_true")
    parser.add_argument("--profile-copy", action="store_true",
                        help="also run three 256 MiB device-to-device copies (a kernel of known traffic, "
                             "to calibrate FETCH_SIZE / WRITE_SIZE counters under rocprofv3)")
    parser.add_argument("--library", default=None,
                        help="another build of libnqhip.so to load (the measuring build that --only encode_phases needs: "
                             "python -m nestquant_aiinfra_amd.build --define NQ_PHASE_STAMPS --output PATH)")
    parser.add_argument("--only", choices=("tpot", "gemm", "attention", "encode", "rowlinear", "encode_phases", "attention_phases",
                                           "gemv_phases", "pair_phases", "prompt"), default=None,
                        help="run one of the extra measurements alone (for profiling) and print its JSON")
    parser.add_argument("--prompt-shape", default=None,
                        help="ROWSxWIDTH: the one prompt shape --only prompt runs (default: 1x128, 8x128 and 1x384)")
    parser.add_argument("--skip-extras", action="store_true",
                        help="only the headline GEMV workload (no prefill GEMM, attention, TPOT)")
    return parser.parse_args()


def hadamard_gpu(x):
    """Normalised Sylvester-Hadamard along the last axis (benchmark input preparation)."""
    import torch
    n = x.shape[-1]
    y = x.reshape(-1, n).float()
    width = 1
    while width < n:
        pairs = y.reshape(-1, n // (2 * width), 2, width)
        y = torch.stack((pairs[:, :, 0] + pairs[:, :, 1], pairs[:, :, 0] - pairs[:, :, 1]), dim=2).reshape(-1, n)
        width *= 2
    return (y / (n ** 0.5)).reshape(x.shape)


def build_workload(device):
    import numpy as np
    import torch
    from nestquant_aiinfra_amd.runtime import w4a4_linear as rt

    per_copy = sum(linear_bytes(1, k, n) for _, k, n, _, _ in SHAPES)
    copies = -(-MIN_ROTATION_BYTES // per_copy)
    cases = []
    for name, k, n, wseed, dseed in SHAPES:
        g = torch.Generator().manual_seed(wseed)
        w = hadamard_gpu((0.02 * torch.randn(n, k, generator=g)).to(device))
        record = rt.quantize_weight_nqrt4(w, q=Q, betas=WEIGHT_BETAS, dither_seed=dseed, tensor_name=name)
        base = rt.prepare_fused_linear(record, device=device)
        weights = [base] + [
            rt.PreparedNQRTLinear(record, None, None,
                                  base.row_norms.clone(), base.beta_table.clone(),
                                  None if base.resolved_words is None else base.resolved_words.clone(),
                                  None if base.resolved_tails is None else base.resolved_tails.clone())
            for _ in range(copies - 1)
        ]
        for m in TOKEN_COUNTS:
            rng = np.random.default_rng(2001 + m)
            x = torch.from_numpy(rng.standard_t(4, size=(m, k)).astype(np.float32)).to(device)
            x = hadamard_gpu(x).to(torch.bfloat16)
            table = torch.tensor(ACTIVATION_BETAS, dtype=torch.float32, device=device)
            cases.append({"name": name, "m": m, "k": k, "n": n, "x": x, "table": table,
                          "weights": weights, "bytes": linear_bytes(m, k, n), "record": record})
    return cases, copies


def run_case(rt, case, copy: int):
    activation = rt.quantize_activation_cuda(case["x"], q=Q, betas=ACTIVATION_BETAS, beta_table=case["table"])
    weight = case["weights"][copy]
    if case["m"] == 1:
        return rt.linear_packed_w4a4_gemv_m1(activation, weight)
    return rt.linear_packed_w4a4_mma_small_m(activation, weight)


def capture_steps(rt, cases, copies):
    """One HIP graph per weight copy; each graph is one step (four encode + linear pairs)."""
    import torch
    stream = torch.cuda.Stream()
    graphs, keep = [], []
    with torch.cuda.stream(stream):
        for case in cases:                       # warm the allocator and load the kernels
            run_case(rt, case, 0)
        stream.synchronize()
        for copy in range(copies):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                keep.append([run_case(rt, case, copy) for case in cases])
            graphs.append(graph)
    torch.cuda.synchronize()
    return graphs, keep, stream


def time_kernel_alone(rt, case, copies, launches_per_graph=None):
    """Average duration of the linear kernel of one case, timed with events around a graph
    of back-to-back launches on the capture stream (weights rotate; activation pre-encoded)."""
    import torch
    activation = rt.quantize_activation_cuda(case["x"], q=Q, betas=ACTIVATION_BETAS, beta_table=case["table"])
    fn = rt.linear_packed_w4a4_gemv_m1 if case["m"] == 1 else rt.linear_packed_w4a4_mma_small_m
    stream = torch.cuda.Stream()
    count = launches_per_graph or copies
    with torch.cuda.stream(stream):
        fn(activation, case["weights"][0])
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            outs = [fn(activation, case["weights"][i % copies]) for i in range(count)]
        for _ in range(3):
            graph.replay()
        stream.synchronize()
        repeats = 10
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record(stream)
        for _ in range(repeats):
            graph.replay()
        end.record(stream)
        end.synchronize()
    del outs
    return begin.elapsed_time(end) * 1e-3 / (repeats * count)


def one_launch_per_case_extra(rt, cases, copies, step_bytes):
    """The headline step with every case's encoder and linear in one launch (`fused_stage_linear`, mode
    "rotated_rows": the form a decode step's pairs run in), one fill per step clearing the flag words: the
    same outputs bit for bit (checked here), time per step from graphs over the same rotating weights."""
    import torch
    device = cases[0]["x"].device
    sync = rt.StageLinearSync(device)

    def one(case, copy):
        return rt.fused_stage_linear(case["x"], [case["weights"][copy]], sync, mode="rotated_rows",
                                     beta_table=case["table"])[0][0]

    same = all(torch.equal(one(case, 0).reshape(-1), run_case(rt, case, 0).reshape(-1)) for case in cases)

    def step(i):
        sync.begin_step()
        return [one(case, i % copies) for case in cases]
    seconds = time_graph(step, copies)
    return {"us_per_step": seconds * 1e6, "GBps": step_bytes / seconds / 1e9, "equals_two_launches": bool(same),
            "waits_ran_out": bool(sync.timed_out)}


def cpu_baseline_torch(cases, budget_s: float):
    """The same four-linear step with whole-tensor torch operations on the CPU, as the reference's own
    CPU path evaluates it: one encode + decode pass per beta over the full tensor, argmin over the
    passes; dither regenerated; dequantise; torch.matmul in FP32."""
    import numpy as np
    import torch
    import oracle
    from oracle import torch_port

    prepared = []
    for case in cases:
        record, n, k = case["record"], case["n"], case["k"]
        codes = oracle.unpack_unsigned(np.frombuffer(record.indices.code_payload, np.uint8), n * k, 4)
        ids = oracle.unpack_unsigned(np.frombuffer(record.indices.beta_payload, np.uint8), n * k // 8, 2)
        prepared.append((case, torch.from_numpy(codes.astype(np.int64)).reshape(n, k // 8, 8),
                         torch.from_numpy(ids.astype(np.int64)).reshape(n, k // 8), record.row_norms.float().cpu(),
                         case["x"].float().cpu()))

    def one_step():
        for case, codes, ids, norms, x in prepared:
            n, k = case["n"], case["k"]
            a_codes, a_ids, a_norms = torch_port.quantize_rows(x, Q, ACTIVATION_BETAS)
            a_hat = torch_port.dequantize_rows(a_codes, a_ids, a_norms, ACTIVATION_BETAS, Q)
            dither = torch_port.dither_stateless(n * k // 8, case["record"].dither_seed).reshape(n, k // 8, 8)
            w_hat = torch_port.dequantize_rows(codes, ids, norms, WEIGHT_BETAS, Q, dither)
            torch.matmul(a_hat, w_hat.t())

    one_step()
    steps, begin = 0, time.perf_counter()
    while True:
        one_step()
        steps += 1
        elapsed = time.perf_counter() - begin
        if elapsed >= budget_s or steps >= 1000:
            break
    step_bytes = sum(case["bytes"] for case in cases)
    return {"value": step_bytes * steps / elapsed / 1e9, "unit": "GB/s", "ms_per_step": elapsed / steps * 1e3,
            "torch_threads": torch.get_num_threads(), "os_cpu_count": os.cpu_count(),
            "sample": f"{steps} full steps of the same four-linear workload in {elapsed:.1f} s "
                      f"(whole-tensor torch operations on the CPU, {torch.get_num_threads()} threads)"}


def cpu_baseline(cases, budget_s: float = 10.0):
    """The CPU oracle on the same workload: NQA4-encode the activation, dequantise the
    NQRT4 weight (dither regenerated), FP32 matvec.  Bounded to about `budget_s` seconds for
    the C restatement and as much again for the torch-vectorised one reported beside it."""
    import numpy as np
    import oracle

    threads = max(1, min(16, len(os.sched_getaffinity(0))))
    oracle.set_num_threads(threads)
    prepared = []
    for case in cases:
        record = case["record"]
        n, k = case["n"], case["k"]
        wc = oracle.unpack_unsigned(np.frombuffer(record.indices.code_payload, np.uint8), n * k, 4)
        wb = oracle.unpack_unsigned(np.frombuffer(record.indices.beta_payload, np.uint8), n * k // 8, 2)
        prepared.append((case, wc, wb, record.row_norms.float().numpy(), case["x"].float().cpu().numpy()))

    def one_step():
        for case, wc, wb, wn, x in prepared:
            ac, ab, an = oracle.quantize_rows(x, Q, ACTIVATION_BETAS)
            a_hat = oracle.dequantize_rows(ac, ab, an, ACTIVATION_BETAS, Q)
            w_hat = oracle.dequantize_rows(wc, wb, wn, WEIGHT_BETAS, Q, seed=case["record"].dither_seed)
            oracle.matmul_nt(a_hat, w_hat)

    one_step()                                   # warm-up (page-in, thread pool)
    steps, begin = 0, time.perf_counter()
    while True:
        one_step()
        steps += 1
        elapsed = time.perf_counter() - begin
        if elapsed >= budget_s or steps >= 1000:
            break
    step_bytes = sum(case["bytes"] for case in cases)
    return {
        "value": step_bytes * steps / elapsed / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"{steps} full steps of the same four-linear workload in {elapsed:.1f} s "
                  f"(C oracle, OpenMP, {threads} threads)",
        "ms_per_step": elapsed / steps * 1e3,
        "torch_vectorised": cpu_baseline_torch(cases, budget_s),
    }


def time_graph(fn, launches: int, repeats: int = 5) -> float:
    """Seconds per call of `fn`, from events around replays of a graph holding `launches` calls."""
    import torch
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        fn(0)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            keep = [fn(i) for i in range(launches)]
        graph.replay()
        stream.synchronize()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record(stream)
        for _ in range(repeats):
            graph.replay()
        end.record(stream)
        end.synchronize()
    del keep
    return begin.elapsed_time(end) * 1e-3 / (repeats * launches)


def prefill_gemm_extra(rt, device):
    """W4A4 prefill linear (MFMA) at gate/up and down shapes, ragged M, outlier-channel inputs."""
    import numpy as np
    import torch
    results = {}
    for name, k, n, wseed, dseed in (("gate_proj", 2048, 8192, 1003, 20261103), ("down_proj", 8192, 2048, 1004, 20261104)):
        g = torch.Generator().manual_seed(wseed)
        w = hadamard_gpu((0.02 * torch.randn(n, k, generator=g)).to(device))
        record = rt.quantize_weight_nqrt4(w, q=Q, betas=WEIGHT_BETAS, dither_seed=dseed, tensor_name=name)
        base = rt.prepare_fused_linear(record, device=device)
        copies = 32
        weights = [base] + [rt.PreparedNQRTLinear(record, None, None,
                                                  base.row_norms, base.beta_table,
                                                  None if base.resolved_words is None else base.resolved_words.clone(),
                                                  None if base.resolved_tails is None else base.resolved_tails.clone())
                            for _ in range(copies - 1)]
        table = torch.tensor(ACTIVATION_BETAS, dtype=torch.float32, device=device)
        for m in (16, 40, 64, 128, 384, 1024, 4096):         # the last two: long prefill, beyond the reference's list
            rng = np.random.default_rng(3001)
            x = rng.standard_normal((m, k)).astype(np.float32)
            x[:, rng.choice(k, size=k // 100, replace=False)] *= 20.0
            x = torch.from_numpy(x).to(device).to(torch.bfloat16)
            activation = rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS, beta_table=table, hadamard=True)
            seconds = time_graph(lambda i: rt.linear_packed_w4a4_mma_chunked_staged(activation, weights[i % copies]), copies)
            encode = time_graph(lambda i: rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS, beta_table=table,
                                                                      hadamard=True), 16)
            flops = 2.0 * m * k * n
            results[f"{name}_m{m}"] = {"us": seconds * 1e6, "TFLOPs": flops / seconds / 1e12,
                                       "mfma_frac": flops / seconds / 2.5e15, "encode_us": encode * 1e6}
        if name == "gate_proj":
            # gate and up of a layer as the model's prefill step launches them: one call for both weights
            g = torch.Generator().manual_seed(wseed + 10)
            w = hadamard_gpu((0.02 * torch.randn(n, k, generator=g)).to(device))
            up_record = rt.quantize_weight_nqrt4(w, q=Q, betas=WEIGHT_BETAS, dither_seed=dseed + 10, tensor_name="up_proj")
            up_base = rt.prepare_fused_linear(up_record, device=device)
            ups = [up_base] + [rt.PreparedNQRTLinear(up_record, None, None, up_base.row_norms, up_base.beta_table,
                                                     up_base.resolved_words.clone(), up_base.resolved_tails.clone())
                               for _ in range(copies - 1)]
            for m in (64, 128, 256, 384):
                rng = np.random.default_rng(3001)
                x = rng.standard_normal((m, k)).astype(np.float32)
                x[:, rng.choice(k, size=k // 100, replace=False)] *= 20.0
                x = torch.from_numpy(x).to(device).to(torch.bfloat16)
                activation = rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS, beta_table=table, hadamard=True)
                seconds = time_graph(lambda i: rt.linear_packed_w4a4_gemm_grouped(
                    activation, [weights[i % copies], ups[i % copies]]), copies)
                flops = 2.0 * m * k * 2 * n
                results[f"gate_up_m{m}"] = {"us": seconds * 1e6, "TFLOPs": flops / seconds / 1e12,
                                            "mfma_frac": flops / seconds / 2.5e15}
            del ups
    return results


def encode_extra(rt, device):
    """E8 row encoder alone: the 2048 x 2048 float32 plumbing case (undithered A4 and dithered
    NQRT4 weight rows) and BF16 activations from one decode row to a long prefill, rotation fused.
    Algorithmic bytes: rows * n * input size + rows * (n / 2 + n / 32 + 4)."""
    import torch
    results = {}
    g = torch.Generator().manual_seed(58)
    cases = [("config1_a4_f32", torch.randn(2048, 2048, generator=g), None, False),
             ("config1_nqrt4_f32", torch.randn(2048, 2048, generator=g), 20261025, False)]
    for m, n in ((1, 2048), (8, 2048), (1, 8192), (8, 8192), (128, 2048), (1024, 2048), (4096, 2048), (4096, 8192)):
        cases.append((f"a4_bf16_m{m}_n{n}", torch.randn(m, n, generator=g).to(torch.bfloat16), None, True))
    act = torch.tensor(ACTIVATION_BETAS, dtype=torch.float32, device=device)
    wgt = torch.tensor(WEIGHT_BETAS, dtype=torch.float32, device=device)
    for name, x, seed, rotate in cases:
        x = x.to(device)
        rows, n = x.shape
        if seed is None:
            fn = lambda i: rt.quantize_rows_packed(x, q=Q, beta_table=act, hadamard=rotate)
        else:
            fn = lambda i: rt.quantize_rows_packed(x, q=Q, beta_table=wgt, dither_seed=seed)
        seconds = time_graph(fn, 16)
        nbytes = rows * n * x.element_size() + rows * (n // 2 + n // 32 + 4)
        results[name] = {"us": seconds * 1e6, "bytes": nbytes, "GBps": nbytes / seconds / 1e9,
                         "hbm_frac": nbytes / seconds / 1e9 / HBM_PEAK_GBPS, "values_per_us": rows * n / seconds / 1e6}
    return results


def encode_phases_extra(rt, device):
    """Where one launch of the decode-size encoder spends its time: the wall-clock stamps that lane 0
    of workgroup 0 leaves at the phase boundaries in a measuring build (--library), beside the
    launch-to-launch time of the same call in a graph.  Nanoseconds; `outside` is what the launch
    costs before the first and after the last stamp of that workgroup."""
    import ctypes
    import torch
    from nestquant_aiinfra_amd import _native
    lib = _native.library()
    if not hasattr(lib, "nq_debug_phase_stamps"):
        sys.exit("bench.py: --only encode_phases needs a library built with --define NQ_PHASE_STAMPS (see --library)")
    lib.nq_debug_phase_stamps.restype = ctypes.c_int
    lib.nq_debug_phase_stamps.argtypes = [ctypes.c_void_p]
    table = torch.tensor(ACTIVATION_BETAS, dtype=torch.float32, device=device)
    g = torch.Generator().manual_seed(59)
    results = {}
    for rows, n in ((1, 2048), (8, 2048), (1, 8192), (8, 8192)):
        x = torch.randn(rows, n, generator=g).to(torch.bfloat16).to(device)
        other = torch.randn(rows, n, generator=g).to(torch.bfloat16).to(device)
        weight = (1.0 + 0.1 * torch.randn(n, generator=g)).to(torch.bfloat16).to(device)
        calls = {
            "plain": lambda: rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS, beta_table=table, hadamard=True),
            "rmsnorm": lambda: rt.fused_input_stage(x, mode="rmsnorm", residual=other, norm_weight=weight, eps=1e-5,
                                                    beta_table=table, want_residual=True),
            "swiglu": lambda: rt.fused_input_stage(x, mode="swiglu", gate=other, beta_table=table),
        }
        for name, call in calls.items():
            seconds = time_graph(lambda i: call(), 16)
            call()
            stamps = (ctypes.c_ulonglong * 16)()
            _native.check(lib.nq_debug_phase_stamps(stamps))
            s = [int(v) * 10 for v in stamps[:12]]                      # 100 MHz ticks -> ns
            inside = s[4] - s[0]
            results[f"{name}_m{rows}_n{n}"] = {
                "launch_ns": round(seconds * 1e9), "outside_ns": round(seconds * 1e9) - inside,
                "stage_ns": s[1] - s[0], "hadamard_ns": s[2] - s[1], "norm_ns": s[3] - s[2], "encode_ns": s[4] - s[3],
                "hadamard_parts_ns": {"registers_and_lanes": s[8] - s[1], "barrier": s[9] - s[8], "lds_passes": s[2] - s[9]},
                "norm_parts_ns": {"chains": s[10] - s[2], "sum_sqrt_divide": s[11] - s[10], "barrier": s[3] - s[11]},
                "encode_parts_ns": {"load_scale_divide": s[5] - s[3], "nearest_point_and_code": s[6] - s[5],
                                    "decode_and_error": s[7] - s[6], "argmin_and_stores": s[4] - s[7]},
            }
    return results


def _rotating_weights(rt, device, name, k, n, wseed, dseed, copies):
    import torch
    g = torch.Generator().manual_seed(wseed)
    w = hadamard_gpu((0.02 * torch.randn(n, k, generator=g)).to(device))
    record = rt.quantize_weight_nqrt4(w, q=Q, betas=WEIGHT_BETAS, dither_seed=dseed, tensor_name=name)
    base = rt.prepare_fused_linear(record, device=device)
    return [base] + [rt.PreparedNQRTLinear(record, None, None, base.row_norms, base.beta_table,
                                           base.resolved_words.clone(), base.resolved_tails.clone())
                     for _ in range(copies - 1)]


def _stamps(lib, entry, count):
    import ctypes
    from nestquant_aiinfra_amd import _native
    if not hasattr(lib, entry):
        sys.exit(f"bench.py: this measurement needs a library built with --define NQ_PHASE_STAMPS (see --library): no {entry}")
    call = getattr(lib, entry)
    call.restype, call.argtypes = ctypes.c_int, [ctypes.c_void_p]
    stamps = (ctypes.c_ulonglong * count)()
    _native.check(call(stamps))
    return [int(v) * 10 for v in stamps]                          # 100 MHz ticks -> ns


def gemv_phases_extra(rt, device):
    """Where one launch of the vector-unit GEMV (resolved weights, one row) spends its time: the
    stamps of lane 0 of workgroup 0 in a measuring build (--library), beside the launch-to-launch
    time of the same call in a graph over weights that rotate through more than the caches hold."""
    import torch
    from nestquant_aiinfra_amd import _native
    lib = _native.library()
    table = torch.tensor(ACTIVATION_BETAS, dtype=torch.float32, device=device)
    results = {}
    for name, k, n, wseed, dseed in SHAPES:
        weights = _rotating_weights(rt, device, name, k, n, wseed, dseed, 48)
        for m in (1, 4):
            x = torch.randn(m, k, generator=torch.Generator().manual_seed(60 + m)).to(torch.bfloat16).to(device)
            activation = rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS, beta_table=table, hadamard=True)
            linear = rt.linear_packed_w4a4_gemv_m1 if m == 1 else rt.linear_packed_w4a4_mma_small_m
            call = lambda i: linear(activation, weights[i % len(weights)])
            seconds = time_graph(call, len(weights))
            flush = torch.empty(128 << 20, dtype=torch.float32, device=device).fill_(1.0)      # cold caches
            torch.cuda.synchronize()
            call(7)
            s = _stamps(lib, "nq_debug_gemv_stamps", 16)
            del flush
            results[f"{name}_m{m}"] = {
                "launch_ns": round(seconds * 1e9), "first_workgroup_ns": s[6] - s[0],
                "setup_and_first_requests_ns": s[1] - s[0], "first_block_decoded_ns": s[2] - s[1],
                "remaining_steps_ns": s[3] - s[2], "lane_sums_ns": s[4] - s[3], "barrier_ns": s[5] - s[4],
                "fold_and_store_ns": s[6] - s[5]}
    return results


def pair_phases_extra(rt, device):
    """The one-launch input stage + linear(s) of a 1B decode step, pair by pair: launch-to-launch time in
    a graph over rotating weights, and the stamps the first and last encoder workgroup and the first and
    last consumer workgroup leave in a measuring build (--library), in ns from the earliest of them."""
    import torch
    from nestquant_aiinfra_amd import _native
    lib = _native.library()
    table = torch.tensor(ACTIVATION_BETAS, dtype=torch.float32, device=device)
    pairs = {"qkv": ("rmsnorm", [(2048, 2048), (512, 2048), (512, 2048)]), "gate_up": ("rmsnorm", [(8192, 2048), (8192, 2048)]),
             "down": ("swiglu", [(2048, 8192)]), "o": ("swiglu", [(2048, 2048)])}
    results, copies = {}, 24
    for name, (mode, shapes) in pairs.items():
        sets = [_rotating_weights(rt, device, f"{name}{i}", k, n, 1100 + i, 20261201 + i, copies) for i, (n, k) in enumerate(shapes)]
        groups = [[members[c] for members in sets] for c in range(copies)]
        k = shapes[0][1]
        for m in (1, 8):
            g = torch.Generator().manual_seed(70 + m)
            x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(device)
            other = torch.randn(m, k, generator=g).to(torch.bfloat16).to(device)
            norm_weight = torch.ones(k, dtype=torch.bfloat16, device=device)
            extra = dict(residual=other, norm_weight=norm_weight, eps=1e-5) if mode == "rmsnorm" else dict(gate=other)
            sync = rt.StageLinearSync(device, sets=256)
            one = lambda i: rt.fused_stage_linear(x, groups[i % copies], sync, mode=mode, beta_table=table, **extra)[0]
            def two(i):
                activation = rt.fused_input_stage(x, mode=mode, beta_table=table, **extra)[0]
                return rt.linear_packed_w4a4_gemv_grouped(activation, groups[i % copies], output_dtype=torch.bfloat16)
            two_launches = time_graph(two, 2 * copies)
            one_launch = time_graph(one, 2 * copies)
            sync.reset()
            flush = torch.empty(128 << 20, dtype=torch.float32, device=device).fill_(1.0)
            torch.cuda.synchronize()
            one(5)
            s = _stamps(lib, "nq_debug_pair_stamps", 32)
            del flush
            origin = min(s[0], s[8], s[16], s[24])
            role = lambda slot, names: {label: s[8 * slot + i] - origin for i, label in enumerate(names)}
            producer = ("start", "encoded", "stores_acknowledged", "behind_barrier")
            consumer = ("start", "weights_decoded", "flags_seen", "multiplied", "stored")
            results[f"{name}_m{m}"] = {
                "two_launches_ns": round(two_launches * 1e9), "one_launch_ns": round(one_launch * 1e9),
                "timed_out": sync.timed_out, "first_encoder": role(0, producer), "last_encoder": role(1, producer),
                "first_consumer": role(2, consumer), "last_consumer": role(3, consumer)}
    return results


def attention_phases_extra(device):
    """Where one launch of the decode attention (stage 1) spends its time, from the wall-clock stamps
    that lane 0 of the first workgroup (row 0, KV head 0, first chunk of pages) leaves in a measuring
    build (--library): contexts of a decode step after a 128-token prompt, and the ragged long ones."""
    import ctypes
    import torch
    from nestquant_aiinfra_amd import _native
    from nestquant_aiinfra_amd.runtime import nqkv
    lib = _native.library()
    if not hasattr(lib, "nq_debug_attention_stamps"):
        sys.exit("bench.py: --only attention_phases needs a library built with --define NQ_PHASE_STAMPS (see --library)")
    lib.nq_debug_attention_stamps.restype = ctypes.c_int
    lib.nq_debug_attention_stamps.argtypes = [ctypes.c_void_p]
    key_betas = tuple(v / 14 for v in (3.50, 4.58, 6.47, 17.06))
    value_betas = tuple(v / 14 for v in (3.53, 5.59, 9.62, 29.03))
    g = torch.Generator().manual_seed(4001)
    results = {}
    for name, lengths in (("decode_after_128", [200] * 8), ("ragged_128_4096", torch.randint(128, 4097, (8,), generator=g).tolist())):
        manager = nqkv.BatchedNQKVCacheManager(capacity=8, num_layers=4, num_kv_heads=8, head_dim=64, max_cache_len=4096,
                                               page_size=16, q=Q, key_betas=key_betas, value_betas=value_betas,
                                               dtype=torch.bfloat16, device=device)
        width = max(lengths)
        for slot in range(8):
            manager.register(slot, slot=slot)
        manager.step_counts.copy_(torch.tensor(lengths, dtype=torch.int32))
        manager.step_active.fill_(True)
        manager.begin_step(rows=8, uniform_count=None)
        for layer in range(4):
            key = hadamard_gpu(torch.randn(8, width, 8, 64, generator=g).to(device)).to(torch.bfloat16)
            value = torch.randn(8, width, 8, 64, generator=g).to(device).to(torch.bfloat16)
            manager.write_layer(layer, key, value)
        query = hadamard_gpu(torch.randn(8, 32, 64, generator=g).to(device)).to(torch.bfloat16)
        slot_ids = torch.arange(8, dtype=torch.int32, device=device)
        active = torch.ones(8, dtype=torch.bool, device=device)
        workspace = nqkv.BatchedNQKVAttentionWorkspace.create(manager.layers[0], batch_size=8, query_heads=32,
                                                              output_dtype=torch.bfloat16)
        call = lambda i: nqkv.launch_nqkv_decode_attention(query, manager.layers[i % 4], slot_ids=slot_ids, active_mask=active,
                                                           attention_scale=0.125, workspace=workspace).clone()
        seconds = time_graph(call, 8)
        call(0)
        stamps = (ctypes.c_ulonglong * 16)()
        _native.check(lib.nq_debug_attention_stamps(stamps))
        s = [int(v) * 10 for v in stamps[:10]]
        results[name] = {"launch_ns_with_merge": round(seconds * 1e9), "tables_ns": s[1] - s[0],
                         "key_requests_and_query_ns": s[2] - s[1], "query_to_registers_ns": s[3] - s[2],
                         "key_pass_ns": s[4] - s[3], "softmax_ns": s[5] - s[4], "value_pass_ns": s[6] - s[5],
                         "fold_and_store_ns": s[7] - s[6], "of_which_fold_ns": s[8] - s[6],
                         "of_which_wait_for_the_workgroup_ns": s[9] - s[8], "inside_ns": s[7] - s[0]}
    return results


def row_linear_extra(rt, device):
    """The BF16 stream kernel: the LM head of the 1B model (128256 x 2048) and, for the optional
    expanded-weights decode, the 1B projection shapes, at 1 and 8 rows.  Algorithmic bytes: the
    BF16 weight once, the activation and the output."""
    import torch
    results = {}
    g = torch.Generator().manual_seed(6100)
    shapes = (("lm_head", 2048, [128256]), ("qkv", 2048, [2048, 512, 512]), ("o_proj", 2048, [2048]),
              ("gate_up", 2048, [8192, 8192]), ("down_proj", 8192, [2048]))
    for name, k, sizes in shapes:
        n = sum(sizes)
        copies = max(2, min(8, (600 << 20) // (n * k * 2)))            # rotate past the 256 MB of last-level cache
        weights = [(0.05 * torch.randn((n, k), generator=g)).to(torch.bfloat16).to(device) for _ in range(copies)]
        for rows in (1, 8):
            act = torch.randn((rows, k), generator=g).to(torch.bfloat16).to(device)
            seconds = time_graph(lambda i: rt.bf16_rows_linear_grouped(act, weights[i % copies], sizes), 2 * copies)
            nbytes = 2 * (n * k + rows * k + rows * n)
            results[f"{name}_m{rows}"] = {"us": seconds * 1e6, "bytes": nbytes, "GBps": nbytes / seconds / 1e9,
                                          "hbm_frac": nbytes / seconds / 1e9 / HBM_PEAK_GBPS}
        del weights
    return results


def rope_gpu(x, positions, theta=500000.0):
    """Llama rotary embedding (rotate-half form) of [..., tokens, heads, dim] rows at `positions` [tokens]."""
    import torch
    dim = x.shape[-1]
    inv_freq = 1.0 / theta ** (torch.arange(0, dim, 2, device=x.device, dtype=torch.float64) / dim)
    angle = positions.to(torch.float64)[:, None] * inv_freq[None, :]
    cos, sin = (torch.cat((f(angle), f(angle)), dim=-1)[:, None, :].float() for f in (torch.cos, torch.sin))
    half = torch.cat((-x[..., dim // 2:], x[..., :dim // 2]), dim=-1)
    return x * cos + half * sin


def attention_extra(device):
    """Paged NQKV4 decode attention: 32 / 8 heads, D 64, batch 8, contexts uniform in [128, 4096],
    RoPE (theta = 500000) on keys and queries before their Hadamard.  Measured on pools that keep the
    decode hints (four more bits per block, the runner's default) and, under `without_hints`, on the six
    streams of the reference's format alone; the algorithmic bytes are those of the six streams either way."""
    results = _attention_measurements(device, hints=True)
    results["without_hints"] = _attention_measurements(device, hints=False)
    return results


def _attention_measurements(device, hints):
    import torch
    from nestquant_aiinfra_amd.runtime import nqkv
    key_betas = tuple(v / 14 for v in (3.50, 4.58, 6.47, 17.06))
    value_betas = tuple(v / 14 for v in (3.53, 5.59, 9.62, 29.03))
    g = torch.Generator().manual_seed(4001)
    lengths = torch.randint(128, 4097, (8,), generator=g).tolist()
    manager = nqkv.BatchedNQKVCacheManager(capacity=8, num_layers=4, num_kv_heads=8, head_dim=64, max_cache_len=4096,
                                           page_size=16, q=Q, key_betas=key_betas, value_betas=value_betas,
                                           dtype=torch.bfloat16, device=device, hints=hints)
    width = max(lengths)
    for slot in range(8):
        manager.register(slot, slot=slot)
    manager.step_counts.copy_(torch.tensor(lengths, dtype=torch.int32))
    manager.step_active.fill_(True)
    manager.begin_step(rows=8, uniform_count=None)
    positions = torch.arange(width, device=device)
    for layer in range(4):                       # distinct layers = distinct (cold) pages per launch
        key = hadamard_gpu(rope_gpu(torch.randn(8, width, 8, 64, generator=g).to(device), positions)).to(torch.bfloat16)
        value = torch.randn(8, width, 8, 64, generator=g).to(device).to(torch.bfloat16)
        manager.write_layer(layer, key, value)
    last = torch.tensor(lengths, device=device) - 1
    query = torch.randn(8, 32, 64, generator=g).to(device)
    query = hadamard_gpu(torch.stack([rope_gpu(query[row:row + 1], last[row:row + 1])[0] for row in range(8)]))
    query = query.to(torch.bfloat16)
    slot_ids = torch.arange(8, dtype=torch.int32, device=device)
    active = torch.ones(8, dtype=torch.bool, device=device)
    workspace = nqkv.BatchedNQKVAttentionWorkspace.create(manager.layers[0], batch_size=8, query_heads=32,
                                                          output_dtype=torch.bfloat16)
    seconds = time_graph(lambda i: nqkv.launch_nqkv_decode_attention(
        query, manager.layers[i % 4], slot_ids=slot_ids, active_mask=active, attention_scale=0.125,
        workspace=workspace).clone(), 8)
    # the first stage alone (the decode step merges its partial results inside the next encoder)
    stage1 = time_graph(lambda i: nqkv.launch_nqkv_decode_attention(
        query, manager.layers[i % 4], slot_ids=slot_ids, active_mask=active, attention_scale=0.125,
        workspace=workspace, merge=False), 8)
    bytes_moved = sum(608 * 16 * (n // 16) + (n % 16) * 8 * 64 * 2 * 2 + 2 * 32 * 64 * 2 for n in lengths)
    step_key = torch.randn(8, 1, 8, 64, device=device).to(torch.bfloat16)
    manager.step_active.fill_(False)             # time the writer's launch without growing the cache
    write = time_graph(lambda i: manager.write_layer(i % 4, step_key, step_key, rotate_keys=True), 8)
    # chunked prefill: the last 128 tokens of every sequence attend causally to the packed cache
    chunk = 128
    chunk_query = hadamard_gpu(torch.randn(8, chunk, 32, 64, generator=g).to(device)).to(torch.bfloat16)
    manager.step_active.fill_(True)
    prefill = time_graph(lambda i: nqkv.nqkv_prefill_attention(
        chunk_query, manager.layers[i % 4], slot_ids=slot_ids, active_mask=active, uniform_count=chunk, scale=0.125), 8)
    prefill_flops = sum(4 * 32 * 64 * sum(n - chunk + t + 1 for t in range(chunk)) for n in lengths)
    # the same chunk with one workgroup per (row, token tile, KV head) walking the whole context, and the
    # longest row alone (one sequence's chunked prefill), with and without the split of the context
    walked = time_graph(lambda i: nqkv.nqkv_prefill_attention(
        chunk_query, manager.layers[i % 4], slot_ids=slot_ids, active_mask=active, uniform_count=chunk, scale=0.125,
        split_context=False), 8)
    longest = max(range(8), key=lambda row: lengths[row])
    one_slot = slot_ids[longest:longest + 1].clone()
    one = {split: time_graph(lambda i: nqkv.nqkv_prefill_attention(
        chunk_query[:1], manager.layers[i % 4], slot_ids=one_slot, active_mask=active[:1], uniform_count=chunk, scale=0.125,
        split_context=split), 8) for split in (True, False)}
    return {"contexts": lengths, "us": seconds * 1e6, "algorithmic_bytes": bytes_moved,
            "GBps": bytes_moved / seconds / 1e9, "hbm_frac": bytes_moved / seconds / 1e9 / HBM_PEAK_GBPS,
            "stage1_us": stage1 * 1e6, "stage1_hbm_frac": bytes_moved / stage1 / 1e9 / HBM_PEAK_GBPS,
            "append_launch_us": write * 1e6,
            "prefill_chunk128": {"us": prefill * 1e6, "flops": prefill_flops,
                                 "TFLOPs": prefill_flops / prefill / 1e12, "us_without_context_split": walked * 1e6,
                                 "longest_row_alone_us": one[True] * 1e6,
                                 "longest_row_alone_us_without_context_split": one[False] * 1e6}}


def engine_tpot(model, capacity, prompt, generate, vocab, generator):
    """The continuous-batching engine at `capacity` slots over `capacity` requests of `prompt` random
    ids and `generate` new tokens each: per-request inter-token wall time, the clock read after a
    device synchronisation at the end of every engine step, so that host scheduling, the graph replay
    and the host argmax are all inside it (the reference's engine harness,
    scripts/benchmark_service_workloads.py:148-151, 215-220)."""
    import torch
    from nestquant_aiinfra_amd.models import llama_w4a4kv4 as asm
    from nestquant_aiinfra_amd.runtime import AdmissionPolicy, ContinuousBatchInferenceEngine, DecodeRequest

    runner = asm.attach_w4a4kv4_cache(model, capacity=capacity, max_cache_len=prompt + generate)
    runner.capture_prefill(rows=capacity, width=prompt)      # the engine admits all `capacity` prompts in its first step
    out = {}
    for name, burst in (("host_sampler", 1), ("device_sampler_burst16", 16)):
        engine = ContinuousBatchInferenceEngine(runner, decode_burst=burst,
                                                admission_policy=AdmissionPolicy(min_prefill_batch=1, max_wait_steps=0))
        engine.initialize()
        requests = [DecodeRequest(f"r{i}", tuple(torch.randint(0, vocab, (prompt,), generator=generator).tolist()), generate)
                    for i in range(capacity)]
        for request in requests:
            engine.submit(request)
        token_times = {request.request_id: [] for request in requests}
        torch.cuda.synchronize()
        started = time.perf_counter()
        while engine.has_work():
            engine.step()
            torch.cuda.synchronize()
            now = time.perf_counter()
            for request in requests:
                times = token_times[request.request_id]
                fresh = len(request.generated_token_ids) - len(times)
                if fresh and not times:
                    times.append(now)
                    fresh -= 1
                if fresh:
                    # the tokens a burst hands over at once are spread evenly over the time since the one before
                    previous = times[-1]
                    times.extend(previous + (now - previous) * (i + 1) / fresh for i in range(fresh))
        wall = time.perf_counter() - started
        gaps = sorted((times[i] - times[i - 1]) * 1e3 for times in token_times.values() for i in range(1, len(times)))
        out[name] = {"tpot_ms_p50": gaps[len(gaps) // 2], "tpot_ms_p95": gaps[int(0.95 * len(gaps))],
                     "tpot_ms_mean": sum(gaps) / len(gaps), "ttft_ms": 1e3 * (min(t[0] for t in token_times.values()) - started),
                     "tokens_per_s": sum(len(t) for t in token_times.values()) / wall}
    return out


def tpot_extra(device, batches=(1, 2, 4, 8), prompt=128, generate=128):
    """Random-init Llama-3.2-1B architecture, all 112 projections W4A4, KV4 cache, captured decode
    step.  Per batch size: mean decode-step wall time (host argmax included), the wall time per
    step when the sampler runs inside the graph (one host read per 64 steps), GPU graph time, and
    the engine's per-request TPOT at that capacity (`engine`)."""
    import tempfile

    import torch
    from transformers import LlamaConfig, LlamaForCausalLM
    from nestquant_aiinfra_amd.models import llama_w4a4kv4 as asm

    torch.manual_seed(5001)
    config = LlamaConfig(hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, num_attention_heads=32,
                         num_key_value_heads=8, head_dim=64, vocab_size=128256, max_position_embeddings=4096,
                         rope_theta=500000.0, tie_word_embeddings=True)
    with torch.device(device):
        model = LlamaForCausalLM(config).to(torch.bfloat16).eval()
    results = {}
    with tempfile.TemporaryDirectory() as folder:
        path = os.path.join(folder, "llama1b_random.nqmc")
        asm.write_w4_checkpoint(model, path)
        packed_bytes = os.path.getsize(path)
        greedy_steps = 64
        runner = asm.build_w4a4kv4_runner(model, path, capacity=max(batches),
                                          max_cache_len=prompt + generate + greedy_steps + 48,
                                          enable_m1_down_splitk=False)
        g = torch.Generator().manual_seed(5002)
        for batch in batches:
            slots = list(range(batch))
            ids = torch.randint(0, config.vocab_size, (batch, prompt), generator=g).to(device)
            # the first prompt of a run also prepares the weights (their resolved form, once per device):
            # it is reported on its own, and the prompt is then run again
            prefill_calls = []
            for _ in range(2):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                logits = runner.prefill_slots(ids, slots=slots, lengths=[prompt] * batch)
                token = logits[:, -1].argmax(-1).reshape(batch, 1)
                torch.cuda.synchronize()
                prefill_calls.append(time.perf_counter() - t0)
                if len(prefill_calls) == 1:
                    del logits
                    runner.release_slots(slots)
            prefill_s = prefill_calls[1]
            # the same prompt again, asking only for the logits the first new token needs
            # (twice: the first call of a shape pays the BLAS library's set-up)
            del logits
            for _ in range(2):
                runner.release_slots(slots)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                logits = runner.prefill_slots(ids, slots=slots, lengths=[prompt] * batch, last_token_logits=True)
                token = logits[:, 0].argmax(-1).reshape(batch, 1)
                torch.cuda.synchronize()
                prefill_last_s = time.perf_counter() - t0
            # and replayed from a captured graph (a single prompt is bound by the host issuing its launches)
            runner.release_slots(slots)
            runner.capture_prefill(rows=batch, width=prompt)
            for _ in range(2):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                logits = runner.prefill_slots(ids, slots=slots, lengths=[prompt] * batch, last_token_logits=True)
                token = logits[:, 0].argmax(-1).reshape(batch, 1)
                torch.cuda.synchronize()
                prefill_graph_s = time.perf_counter() - t0
                if _ == 0:
                    runner.release_slots(slots)
            if not runner.graph_captured:
                runner.capture()
            position = torch.full((batch, 1), prompt, dtype=torch.long, device=device)
            step_times = []
            for _ in range(generate):
                t0 = time.perf_counter()
                out = runner.decode(token, slots=slots, positions=position)
                token = out[:, 0].argmax(-1).reshape(batch, 1)
                token.tolist()                                   # host sampler read, as the reference's engine does
                step_times.append(time.perf_counter() - t0)
                position = position + 1
            torch.cuda.synchronize()
            t0 = time.perf_counter()                             # sampler inside the graph, one host read at the end
            runner.decode_greedy(token, slots=slots, positions=position, steps=greedy_steps).tolist()
            greedy_s = (time.perf_counter() - t0) / greedy_steps
            width = next(w for w in sorted(runner._graphs) if w >= batch)
            graph = runner._graphs[width][0]
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()                                       # rows stay active: 20 more tokens per slot
            for _ in range(20):
                graph.replay()
            end.record()
            end.synchronize()
            runner.release_slots(slots)
            steps = sorted(step_times[1:])
            results[f"batch{batch}"] = {
                "tpot_ms_mean": 1e3 * sum(steps) / len(steps), "tpot_ms_p50": 1e3 * steps[len(steps) // 2],
                "tpot_ms_p95": 1e3 * steps[int(0.95 * len(steps))], "graph_replay_ms": begin.elapsed_time(end) / 20,
                "tpot_ms_device_sampler": greedy_s * 1e3,
                "prefill_ms": prefill_s * 1e3, "prefill_ms_first_call": prefill_calls[0] * 1e3, "prefill_ms_last_token_logits": prefill_last_s * 1e3,
                "prefill_ms_last_token_logits_captured": prefill_graph_s * 1e3, "tokens_per_s": batch / (sum(steps) / len(steps)),
                "tokens_per_s_device_sampler": batch / greedy_s,
            }
        # the same decode with BF16 copies of the projection weights kept beside the packed ones
        # (16 instead of 6 bits per weight in HBM; the step streams them instead of decoding)
        runner.fused_step.expand_weights = True
        runner._graphs.clear()
        for batch in batches:
            slots = list(range(batch))
            ids = torch.randint(0, config.vocab_size, (batch, prompt), generator=g).to(device)
            logits = runner.prefill_slots(ids, slots=slots, lengths=[prompt] * batch, last_token_logits=True)
            token = logits[:, 0].argmax(-1).reshape(batch, 1)
            if not runner.graph_captured:
                runner.capture()
            position = torch.full((batch, 1), prompt, dtype=torch.long, device=device)
            runner.decode_greedy(token, slots=slots, positions=position, steps=generate)       # to the same context
            position = position + generate
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            runner.decode_greedy(token, slots=slots, positions=position, steps=greedy_steps).tolist()
            greedy_s = (time.perf_counter() - t0) / greedy_steps
            runner.release_slots(slots)
            results[f"batch{batch}"]["tpot_ms_device_sampler_expanded_weights"] = greedy_s * 1e3
        runner.fused_step.expand_weights = False
        for batch in batches:
            results[f"batch{batch}"]["engine"] = engine_tpot(model, batch, prompt, generate, config.vocab_size, g)
        results["expanded_weight_bytes"] = sum(
            sum(t.numel() * 2 for t in entry if isinstance(t, torch.Tensor))
            for entry in runner.fused_step._expanded.values() if entry is not None)
        results["checkpoint_bytes"] = packed_bytes
    return results


def prompt_extra(device, shapes=((1, 128), (8, 128), (1, 384)), repeats=10):
    """Prompts into empty slots of the random-init Llama-3.2-1B runner, replayed from their captured graphs
    (the last token's logits only, as an engine asks for them): median GPU time from the first host
    operation of `prefill_slots` to the end of the graph, and the wall time to the sampled token.
    The mode a kernel trace of a prompt is taken from."""
    import tempfile

    import torch
    from transformers import LlamaConfig, LlamaForCausalLM
    from nestquant_aiinfra_amd.models import llama_w4a4kv4 as asm

    torch.manual_seed(5001)
    config = LlamaConfig(hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, num_attention_heads=32,
                         num_key_value_heads=8, head_dim=64, vocab_size=128256, max_position_embeddings=4096,
                         rope_theta=500000.0, tie_word_embeddings=True)
    with torch.device(device):
        model = LlamaForCausalLM(config).to(torch.bfloat16).eval()
    results = {}
    with tempfile.TemporaryDirectory() as folder:
        path = os.path.join(folder, "llama1b_random.nqmc")
        asm.write_w4_checkpoint(model, path)
        runner = asm.build_w4a4kv4_runner(model, path, capacity=max(rows for rows, _ in shapes),
                                          max_cache_len=max(width for _, width in shapes) + 64)
        g = torch.Generator().manual_seed(5003)
        for rows, width in shapes:
            ids = torch.randint(0, config.vocab_size, (rows, width), generator=g).to(device)
            slots = list(range(rows))
            for _ in range(2):                               # the first prompt also prepares the weights
                runner.prefill_slots(ids, slots=slots, lengths=[width] * rows, last_token_logits=True)
                runner.release_slots(slots)
            runner.capture_prefill(rows=rows, width=width)
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            gpu_ms, wall_ms = [], []
            for _ in range(repeats):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                begin.record()
                logits = runner.prefill_slots(ids, slots=slots, lengths=[width] * rows, last_token_logits=True)
                end.record()
                logits[:, 0].argmax(-1).tolist()
                wall_ms.append((time.perf_counter() - t0) * 1e3)
                gpu_ms.append(begin.elapsed_time(end))
                runner.release_slots(slots)
            results[f"{rows}x{width}"] = {"gpu_ms_p50": sorted(gpu_ms)[len(gpu_ms) // 2],
                                          "wall_ms_to_token_p50": sorted(wall_ms)[len(wall_ms) // 2],
                                          "graph_replays": runner.prefill_graph_replay_counts[(rows, width)]}
    return results


MFMA_BF16_PEAK_TFLOPS = 2500.0


def extra_rooflines(extra):
    """One roofline object per secondary kernel, from the measurements already taken: the prefill
    GEMM at 128, 384 and 4096 rows against the dense BF16 matrix-core peak, decode attention and the
    decode-size encoder against HBM."""
    def gemm_object(name, m, note):
        row = extra["prefill_gemm"][f"{name}_m{m}"]
        k, n = (2048, 8192) if name == "gate_proj" else (8192, 2048)
        return {"bound": "mfma", "workload": f"{name} K{k} N{n} M{m} ({note})", "achieved": row["TFLOPs"],
                "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": row["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS,
                "launch_us": row["us"]}
    fused, once = "weight decoded inside the product's launch", "decode of the weight included"
    encoders = {name: extra["e8_encode"][name] for name in ("a4_bf16_m1_n2048", "a4_bf16_m1_n8192", "a4_bf16_m4096_n8192")}
    attention = extra["nqkv_attention"]
    return {
        # the reference's own prefill row counts (128 and 384 rows), then a long prompt
        "prefill_gemm": gemm_object("gate_proj", 128, fused),
        "prefill_gemm_m384": gemm_object("gate_proj", 384, once),
        "prefill_gemm_gate_up_m128": {
            "bound": "mfma", "workload": "gate_proj + up_proj K2048 N2x8192 M128 in one launch, as the prefill step runs them",
            "achieved": extra["prefill_gemm"]["gate_up_m128"]["TFLOPs"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": extra["prefill_gemm"]["gate_up_m128"]["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS,
            "launch_us": extra["prefill_gemm"]["gate_up_m128"]["us"]},
        "prefill_gemm_down_m128": gemm_object("down_proj", 128, fused),
        "prefill_gemm_down_m384": gemm_object("down_proj", 384, once),
        "prefill_gemm_m4096": gemm_object("gate_proj", 4096, once),
        "nqkv_attention": {"bound": "hbm", "workload": "batch 8, 32 / 8 heads, D 64, contexts uniform in [128, 4096]",
                           "achieved": attention["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                           "frac": attention["hbm_frac"], "launch_us": attention["us"],
                           "algorithmic_bytes": attention["algorithmic_bytes"],
                           "stage1_launch_us": attention["stage1_us"], "stage1_frac": attention["stage1_hbm_frac"]},
        "e8_encode": {name: {"bound": "hbm", "achieved": row["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                             "frac": row["hbm_frac"], "launch_us": row["us"], "algorithmic_bytes": row["bytes"]}
                      for name, row in encoders.items()},
    }


def main() -> None:
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only; run with --gpus 1 "
                 "(nothing in the path uses a second GPU)")
    if args.library:
        os.environ["NQHIP_LIBRARY"] = str(Path(args.library).resolve())
    import torch
    from nestquant_aiinfra_amd import _native
    from nestquant_aiinfra_amd.runtime import w4a4_linear as rt

    _native.library()                            # fail loudly if the HIP library is missing
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    if args.profile_copy:
        source = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=device).fill_(1)
        target = torch.empty_like(source)
        for _ in range(3):
            target.copy_(source)                 # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del source, target

    if args.only:
        extra = {"tpot": lambda: tpot_extra(device), "gemm": lambda: prefill_gemm_extra(rt, device),
                 "attention": lambda: attention_extra(device), "encode": lambda: encode_extra(rt, device),
                 "rowlinear": lambda: row_linear_extra(rt, device),
                 "encode_phases": lambda: encode_phases_extra(rt, device),
                 "attention_phases": lambda: attention_phases_extra(device),
                 "gemv_phases": lambda: gemv_phases_extra(rt, device),
                 "pair_phases": lambda: pair_phases_extra(rt, device),
                 "prompt": lambda: prompt_extra(device, **(
                     {"shapes": (tuple(int(v) for v in args.prompt_shape.split("x")),)} if args.prompt_shape else {}))
                 }[args.only]()
        print(json.dumps({args.only: extra}))
        return

    cases, copies = build_workload(device)
    graphs, keep, stream = capture_steps(rt, cases, copies)
    step_bytes = sum(case["bytes"] for case in cases)

    with torch.cuda.stream(stream):
        for i in range(args.warmup):
            graphs[i % copies].replay()
        torch.cuda.synchronize()
        begin = time.perf_counter()
        for i in range(args.steps):
            graphs[(args.warmup + i) % copies].replay()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - begin

    per_case = {}
    for case in cases:
        seconds = time_kernel_alone(rt, case, copies)
        per_case[f"{case['name']}_m{case['m']}"] = {
            "us": seconds * 1e6, "bytes": case["bytes"], "GBps": case["bytes"] / seconds / 1e9,
            "hbm_frac": case["bytes"] / seconds / 1e9 / HBM_PEAK_GBPS,
        }
    dominant = max(per_case, key=lambda name: per_case[name]["us"])
    roofline = {
        "bound": "hbm", "kernel": f"{CASE_KERNEL.get(dominant, 'w4a4_gemv_kernel')} ({dominant})",
        "achieved": per_case[dominant]["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": per_case[dominant]["GBps"] / HBM_PEAK_GBPS, "traffic": measured_traffic_bytes(dominant),
        "launch_us": per_case[dominant]["us"], "algorithmic_bytes": per_case[dominant]["bytes"],
    }

    result = {
        "metric": "w4a4_decode_gemv_algorithmic_GBps", "value": step_bytes * args.steps / elapsed / 1e9,
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": "W4A4 decode linear: q_proj K2048 N2048 + down_proj K8192 N2048, M=1 and M=8, "
                        "NQA4 encode on GPU + packed linear per case, cold weights (rotating copies)",
            "weight_copies": copies, "step_algorithmic_bytes": step_bytes,
        },
        "roofline": roofline,
        "cpu_baseline": None if args.skip_cpu_baseline else cpu_baseline(cases),
        "extra": {"linear_kernel_alone": per_case},
    }
    if not args.skip_extras:
        del graphs, keep
        result["extra"]["one_launch_per_case"] = one_launch_per_case_extra(rt, cases, copies, step_bytes)
        for case in cases:
            case["weights"] = case["weights"][:1]
        torch.cuda.empty_cache()
        result["extra"]["e8_encode"] = encode_extra(rt, device)
        result["extra"]["prefill_gemm"] = prefill_gemm_extra(rt, device)
        result["extra"]["nqkv_attention"] = attention_extra(device)
        result["extra"]["bf16_row_linear"] = row_linear_extra(rt, device)
        result["extra"]["llama_1b_w4a4kv4"] = tpot_extra(device)
        result["extra"]["rooflines"] = extra_rooflines(result["extra"])
    print(json.dumps(result))


if __name__ == "__main__":
    main()
