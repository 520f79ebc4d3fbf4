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


def parse_args() -> argparse.Namespace:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=200)
    parser.add_argument("--warmup", type=int, default=20)
    parser.add_argument("--skip-cpu-baseline", action="store_true")
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
            rt.PreparedNQRTLinear(record, base.code_payload.clone(), base.beta_payload.clone(),
                                  base.row_norms.clone(), base.beta_table.clone())
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


def cpu_baseline(cases, budget_s: float = 20.0):
    """The CPU oracle on the same workload: NQA4-encode the activation, dequantise the
    NQRT4 weight (dither regenerated), FP32 matvec.  Bounded to about `budget_s` seconds."""
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
        if elapsed >= budget_s or steps >= 50:
            break
    step_bytes = sum(case["bytes"] for case in cases)
    return {
        "value": step_bytes * steps / elapsed / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"{steps} full steps of the same four-linear workload in {elapsed:.1f} s "
                  f"(C oracle, OpenMP, {threads} threads)",
        "ms_per_step": elapsed / steps * 1e3,
    }


def main() -> None:
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only; run with --gpus 1 "
                 "(nothing in the path uses a second GPU)")
    import torch
    from nestquant_aiinfra_amd import _native
    from nestquant_aiinfra_amd.runtime import w4a4_linear as rt

    _native.library()                            # fail loudly if the HIP library is missing
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

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
        "bound": "hbm", "kernel": f"w4a4_gemv_kernel ({dominant})",
        "achieved": per_case[dominant]["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": per_case[dominant]["GBps"] / HBM_PEAK_GBPS, "traffic": None,
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
    print(json.dumps(result))


if __name__ == "__main__":
    main()
