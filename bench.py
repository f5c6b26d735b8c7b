"""Benchmark of the MoE hot path on one MI355X.

A "step" is one forward + backward pass of the Mixtral-shaped MoE layer (bf16 with fp32
accumulation, hidden 4096, per-expert intermediate 14336, 8 experts, top-2, 8192 tokens) over
synthetic inputs that are already resident in HBM.  Prints ONE JSON line with the whole-job
throughput in tokens/s, the roofline position of the dominant kernel (timed with events on the
launch stream during the timed steps) and a CPU baseline: the torch restatement of the
reference's torch path (oracle/torch_oracle.py) timed on this host's cores on a bounded sample.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-aux]
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks (dense)
PEAK_BF16_FLOPS = 2.5e15
PEAK_FP16_FLOPS = 2.5e15
PEAK_FP32_MATRIX_FLOPS = 157.3e12
PEAK_HBM_BYTES = 8.0e12

# HBM-side bytes per launch of the grouped GEMM kernels at this workload are not measured by this script: they come
# from two rocprofv3 --pmc runs of it (FETCH_SIZE, WRITE_SIZE), whose per-kernel averages and copy-kernel scale
# factors are kept in the profile summary below.  `roofline.traffic` is read from that file at run time.
TRAFFIC_PROFILE = os.path.join("profiles", "moe_c2_bench_rocprofv3.txt")
TRAFFIC_ROW_TAGS = {
    (2, 0): "xma_grouped_gemm/MT",
    (0, 1): "xma_grouped_gemm/TN+swiglu",
    (0, 0): "xma_grouped_gemm/TN",
    (1, 2): "xma_grouped_gemm/NN+swiglu_bwd",
    (1, 0): "xma_grouped_gemm/NN",
}


def _profile_blob_id() -> str | None:
    """git blob id (sha1 of 'blob <size>\\0' + contents) of the profile summary the traffic figure is read from, so
    that a reader can tell which revision of the file a result line used; None if the file is absent."""

    import hashlib

    try:
        data = open(os.path.join(ROOT, TRAFFIC_PROFILE), "rb").read()
    except OSError:
        return None
    return hashlib.sha1(b"blob %d\0" % len(data) + data).hexdigest()


def _profiled_traffic_bytes() -> dict:
    """tag -> HBM-side bytes per launch, from the table 'layout,epi  FETCH KiB  WRITE KiB' of the profile summary
    and the scale factors it states ('FETCH_SIZE is scaled by F and WRITE_SIZE by W'); {} if the file is absent."""

    import re

    try:
        text = open(os.path.join(ROOT, TRAFFIC_PROFILE), encoding="utf-8").read()
    except OSError:
        return {}
    scale = re.search(r"FETCH_SIZE is scaled by ([0-9.]+) and WRITE_SIZE by ([0-9.]+)", text)
    if scale is None:
        return {}
    fetch_scale, write_scale = float(scale.group(1)), float(scale.group(2))
    out = {}
    for layout, epi, fetch_kib, write_kib in re.findall(r"^\s*(\d),\s*(\d)\s+(\d+)\s+(\d+)\s", text, flags=re.M):
        tag = TRAFFIC_ROW_TAGS.get((int(layout), int(epi)))
        if tag is not None:
            out[tag] = (int(fetch_kib) * fetch_scale + int(write_kib) * write_scale) * 1024
    return out

WORKLOAD = {
    "workload": "Mixtral-shaped MoE layer, forward+backward",
    "tokens": 8192,
    "hidden": 4096,
    "intermediate": 14336,
    "experts": 8,
    "top_k": 2,
    "activation": "swiglu_packed",
    "routing": "linear gate, near-uniform expert load",
}


# The other two GPU configurations of the workload definition.  They are timed after the headline region and
# reported under "other_configs"; the headline line stays the Mixtral-shaped layer.
OTHER_WORKLOADS = [
    {
        "workload": "fine-grained MoE layer, forward+backward",
        "tokens": 16384, "hidden": 2048, "intermediate": 1024, "experts": 64, "top_k": 6,
        "activation": "swiglu_packed", "routing": "linear gate, near-uniform expert load",
    },
    {
        "workload": "skewed-routing MoE layer, forward+backward",
        "tokens": 16384, "hidden": 2048, "intermediate": 768, "experts": 128, "top_k": 8,
        "activation": "swiglu_packed",
        "routing": "linear gate + bias[e] = -c * 1.2 * ln(e + 1); c raised from 1 in steps of 0.5 until >= 4 experts are empty",
    },
]  # fmt: skip


def _parse() -> argparse.Namespace:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-aux", action="store_true", help="skip the stand-alone timings of the HBM-bound kernels")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the fine-grained and skewed-routing layers")
    ap.add_argument("--other-steps", type=int, default=10, help="timed passes of each of the other configurations")
    ap.add_argument("--no-other-dtypes", action="store_true", help="skip the fp16 and fp32 passes of the same layer")
    ap.add_argument("--no-library-gemm", action="store_true", help="skip the loop of library GEMMs of the same shapes")
    ap.add_argument("--only-config", choices=["fine-grained", "skewed"], default=None,
                    help="run only that one of the other configurations (the command its profile is taken with)")
    ap.add_argument("--library-gemm-only", action="store_true",
                    help="run only the loop of library GEMMs (the command the library's counter profile is taken with)")
    ap.add_argument("--reduction-sweep", action="store_true",
                    help="run only the sweep over the reduction length that separates a tile's fixed cost from its "
                    "cost per reduction step, for the grouped kernel and for the library's dense GEMM")
    ap.add_argument("--cpu-sample-tokens", type=int, default=8192)
    ap.add_argument(
        "--copy-probe",
        action="store_true",
        help="also run one plain 1 GiB device copy, the known-size kernel that scales rocprofv3's FETCH_SIZE / WRITE_SIZE",
    )
    return ap.parse_args()


def _cpu_baseline(moe, x, d_y, sample_tokens: int) -> dict:
    """Reference torch path on the host cores, same layer, first `sample_tokens` tokens."""

    import torch

    from oracle import torch_oracle as to

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    k = moe.top_k
    params = [p.detach().cpu().requires_grad_() for p in (moe.gate.weight, moe.c_fc.weight, moe.c_proj.weight)]
    sample_tokens = min(sample_tokens, x.size(0))
    xs = x.detach()[:sample_tokens].cpu().requires_grad_()
    dys = d_y[:sample_tokens].cpu()

    def step() -> float:
        t0 = time.perf_counter()
        y, _ = to.moe_forward(xs, params[0], params[1], params[2], k)
        y.backward(dys)
        dt = time.perf_counter() - t0
        xs.grad = None
        for p in params:
            p.grad = None
        return dt

    step()  # warm-up
    seconds = step()
    return {
        "value": sample_tokens / seconds,
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"first {sample_tokens} of {x.size(0)} tokens of the same layer and dtype, forward+backward, "
        f"1 timed iteration after 1 warm-up ({seconds:.2f} s); per-expert weight-gradient zero fills do not "
        "shrink with the sample, so the full-size rate is no lower than this",
    }


def _kernel_table(summary: dict, steps: int) -> list:
    """Per-kernel rows (average launch time, work rate, fraction of the bounding peak) from a Timeline summary."""

    kernels = []
    for tag, row in sorted(summary.items(), key=lambda kv: -kv[1]["ms"]):
        avg_ms = row["ms"] / row["launches"]
        entry = {
            "kernel": tag,
            "launches_per_step": row["launches"] / steps,
            "avg_ms": round(avg_ms, 4),
            "ms_per_step": round(row["ms"] / steps, 4),
        }
        if row["flops"] > 0:
            entry["flops_per_launch"] = row["flops"] / row["launches"]
            entry["tflops"] = round(row["flops"] / row["ms"] / 1e9, 2)
            entry["frac_of_bf16_peak"] = round(row["flops"] / (row["ms"] * 1e-3) / PEAK_BF16_FLOPS, 4)
        elif row["bytes"] > 0:
            entry["gbps"] = round(row["bytes"] / row["ms"] / 1e6, 1)
            entry["frac_of_hbm_peak"] = round(row["bytes"] / (row["ms"] * 1e-3) / PEAK_HBM_BYTES, 4)
        kernels.append(entry)
    return kernels


def _other_config(workload: dict, steps: int, warmup: int) -> dict:
    """Forward+backward of one of OTHER_WORKLOADS, timed like the headline region (host clock around `steps`
    passes, events on the launch stream around every native call)."""

    import math

    import torch

    import flash_model_architectures_amd as xma
    from flash_model_architectures_amd import _native
    from flash_model_architectures_amd.utils import skewed_router_bias

    dev, dt = torch.device("cuda:0"), torch.bfloat16
    T, H, I = workload["tokens"], workload["hidden"], workload["intermediate"]
    E, k = workload["experts"], workload["top_k"]
    torch.manual_seed(0)
    moe = xma.MoE(E, k, H, I, xma.swiglu_packed, True, False, 0.02).to(dt).to(dev)
    x = torch.randn(T, H, device=dev).to(dt).requires_grad_()
    d_y = torch.randn(T, H, device=dev).to(dt)

    result = {"config": workload}
    if "bias" in workload["routing"]:
        with torch.no_grad():
            raw = moe.gate(x)
        bias, c = skewed_router_bias(raw, k)
        moe.gate.register_forward_hook(lambda mod, inp, out: out + bias)
        result["zipf_bias_scale_c"] = c

    def step() -> None:
        y, _ = moe(x)
        y.backward(d_y)
        x.grad = None
        moe.zero_grad(set_to_none=True)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    timeline = _native.Timeline()
    _native.set_timeline(timeline)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    _native.set_timeline(None)

    with torch.no_grad():
        logits = moe.gate(x)
        _, selected = xma.topk_softmax(logits, k)
        counts = xma.route_tokens(selected, E).expert_frequency.cpu().to(torch.int64)
        # tokens whose k-th and (k+1)-th largest router logits are equal: the only place where the choice of
        # experts rests on a tie rule (lower expert index here)
        ranked = torch.sort(logits.float(), dim=-1, descending=True).values
        ties = int((ranked[:, k - 1] == ranked[:, k]).sum()) if E > k else 0
    kernels = _kernel_table(timeline.summary(), steps)
    gemm_ms = sum(kr["ms_per_step"] for kr in kernels if kr["kernel"].startswith("xma_grouped_gemm"))
    flops = 18.0 * T * k * H * I
    ms_per_step = seconds / steps * 1e3
    result.update(
        {
            "tokens_per_s": round(T * steps / seconds, 1),
            "ms_per_step": round(ms_per_step, 3),
            "steps": steps,
            "layer_tflops": round(flops / (ms_per_step * 1e-3) / 1e12, 2),
            "grouped_gemm_ms_per_step": round(gemm_ms, 4),
            "grouped_gemm_tflops": round(flops / (gemm_ms * 1e-3) / 1e12, 2) if gemm_ms else None,
            "grouped_gemm_frac_of_bf16_peak": round(flops / (gemm_ms * 1e-3) / PEAK_BF16_FLOPS, 4) if gemm_ms else None,
            "expert_rows": {
                "routed_rows": int(counts.sum()),
                "empty_experts": int((counts == 0).sum()),
                "min": int(counts.min()),
                "max": int(counts.max()),
                "experts_under_256_rows": int((counts < 256).sum()),
                "row_tiles_of_256": int(sum(math.ceil(c / 256) for c in counts.tolist())),
                "per_expert": counts.tolist(),
            },
            "tokens_with_a_tie_at_the_selection_boundary": ties,
            "kernels": kernels,
        }
    )
    return result


def _other_dtype(dtype_name: str, steps: int, warmup: int) -> dict:
    """The headline layer (same shape, same seed) in another element type: fp16 through the same LDS-DMA kernels as
    bf16, fp32 through the register-staged kernel with true-fp32 matrix instructions.  Timed like the headline region."""

    import torch

    import flash_model_architectures_amd as xma
    from flash_model_architectures_amd import _native

    dt, peak = {"fp16": (torch.float16, PEAK_FP16_FLOPS), "fp32": (torch.float32, PEAK_FP32_MATRIX_FLOPS)}[dtype_name]
    dev = torch.device("cuda:0")
    T, H, I = WORKLOAD["tokens"], WORKLOAD["hidden"], WORKLOAD["intermediate"]
    E, k = WORKLOAD["experts"], WORKLOAD["top_k"]
    torch.manual_seed(0)
    moe = xma.MoE(E, k, H, I, xma.swiglu_packed, True, False, 0.02).to(dt).to(dev)
    x = torch.randn(T, H, device=dev).to(dt).requires_grad_()
    d_y = torch.randn(T, H, device=dev).to(dt)

    def step() -> None:
        y, _ = moe(x)
        y.backward(d_y)
        x.grad = None
        moe.zero_grad(set_to_none=True)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    timeline = _native.Timeline()
    _native.set_timeline(timeline)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    _native.set_timeline(None)
    kernels = _kernel_table(timeline.summary(), steps)
    for kr in kernels:  # the table's fraction column assumes the bf16 peak
        if "tflops" in kr:
            kr["frac_of_matrix_peak"] = round(kr["tflops"] * 1e12 / peak, 4)
            kr.pop("frac_of_bf16_peak", None)
    gemm_ms = sum(kr["ms_per_step"] for kr in kernels if kr["kernel"].startswith("xma_grouped_gemm"))
    flops = 18.0 * T * k * H * I
    ms_per_step = seconds / steps * 1e3
    return {
        "dtype": dtype_name,
        "matrix_peak_tflops": peak / 1e12,
        "tokens_per_s": round(T * steps / seconds, 1),
        "ms_per_step": round(ms_per_step, 3),
        "steps": steps,
        "grouped_gemm_ms_per_step": round(gemm_ms, 4),
        "grouped_gemm_tflops": round(flops / (gemm_ms * 1e-3) / 1e12, 2) if gemm_ms else None,
        "grouped_gemm_frac_of_matrix_peak": round(flops / (gemm_ms * 1e-3) / peak, 4) if gemm_ms else None,
        "kernels": [kr for kr in kernels if kr["kernel"].startswith("xma_grouped_gemm")],
    }


def _library_gemms(T: int, H: int, I: int, E: int, k: int, iters: int = 3) -> dict:
    """The six GEMM groups of a pass as a loop of LIBRARY GEMMs (torch.matmul -> hipBLASLt), one per expert, every
    expert holding M / E rows, random bf16 operands: no ragged groups, no gather / scatter, no fused activation.  A
    comparison figure for the grouped kernels, measured on the same device in the same run."""

    import torch

    dev, dt = "cuda", torch.bfloat16
    rows = T * k // E
    g = torch.Generator(device=dev).manual_seed(1)
    mk = lambda *shape: torch.randn(*shape, device=dev, generator=g).to(dt)
    x, a, dy, dh = mk(rows, H), mk(rows, I), mk(rows, H), mk(rows, 2 * I)
    w1, w2 = mk(E, 2 * I, H), mk(E, H, I)
    groups = {
        "up projection [M/E,H] x [2I,H]^T": (lambda e: torch.matmul(x, w1[e].t()), 2.0 * rows * 2 * I * H),
        "down projection [M/E,I] x [H,I]^T": (lambda e: torch.matmul(a, w2[e].t()), 2.0 * rows * I * H),
        "d act [M/E,H] x [H,I]": (lambda e: torch.matmul(dy, w2[e]), 2.0 * rows * I * H),
        "dX [M/E,2I] x [2I,H]": (lambda e: torch.matmul(dh, w1[e]), 2.0 * rows * 2 * I * H),
        "dW up [M/E,2I]^T x [M/E,H]": (lambda e: torch.matmul(dh.t(), x), 2.0 * rows * 2 * I * H),
        "dW down [M/E,H]^T x [M/E,I]": (lambda e: torch.matmul(dy.t(), a), 2.0 * rows * I * H),
    }
    out, total_ms, total_flops = [], 0.0, 0.0
    for name, (fn, flops) in groups.items():
        for e in range(E):
            fn(e)
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            for e in range(E):
                fn(e)
        end.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(end) / iters
        total_ms += ms
        total_flops += flops * E
        out.append({"gemm": name, "ms_all_experts": round(ms, 4), "tflops": round(flops * E / ms / 1e9, 1),
                    "frac_of_bf16_peak": round(flops * E / (ms * 1e-3) / PEAK_BF16_FLOPS, 4)})
    # and ONE dense GEMM per projection over all M routed rows with a single expert's weights: the same FLOPs as the
    # grouped launch with no group structure at all, i.e. what the library reaches when nothing is ragged
    xa, aa = mk(T * k, H), mk(T * k, I)
    dense = []
    for name, fn, flops in (
        ("dense [M,H] x [2I,H]^T", lambda: torch.matmul(xa, w1[0].t()), 2.0 * T * k * 2 * I * H),
        ("dense [M,I] x [H,I]^T", lambda: torch.matmul(aa, w2[0].t()), 2.0 * T * k * I * H),
    ):
        fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        end.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(end) / iters
        dense.append({"gemm": name, "ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1),
                      "frac_of_bf16_peak": round(flops / (ms * 1e-3) / PEAK_BF16_FLOPS, 4)})
    return {
        "what": f"{E} library GEMMs per group, {rows} rows each, bf16, random operands (torch.matmul)",
        "ms_per_pass": round(total_ms, 3),
        "frac_of_bf16_peak": round(total_flops / (total_ms * 1e-3) / PEAK_BF16_FLOPS, 4),
        "groups": out,
        "single_dense_gemm_of_the_same_size": dense,
    }


def _reduction_sweep(M: int = 16384, N: int = 16384, E: int = 8, iters: int = 8) -> dict:
    """[M, K] x [N, K]^T in bf16 with M / E rows per expert (no ragged tiles, identity row map) for a range of
    reduction lengths K, with the grouped kernel and with one dense library GEMM of the same size.  M x N is a whole
    number of rounds of 256 tiles of 256 x 256, so the time of a round is a straight line in K: its slope is what
    the main loop costs, its intercept what a tile costs outside the loop (finding the tile, first loads, epilogue,
    the hand-over to the next work-group)."""

    import numpy as np
    import torch

    from flash_model_architectures_amd import ops

    dev, dt = "cuda", torch.bfloat16
    rounds = (M // 256) * (N // 256) / 256.0
    offsets = torch.arange(0, M + 1, M // E, dtype=torch.int32, device=dev)
    rows = torch.arange(M, dtype=torch.int32, device=dev)
    expert_of_row = torch.repeat_interleave(torch.arange(E, device=dev), M // E).int()
    out = torch.empty(M, N, device=dev, dtype=dt)

    def timed(fn) -> float:
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / iters * 1e3  # microseconds

    points = []
    for K in (1024, 2048, 4096, 8192, 14336):
        a = torch.randn(M, K, device=dev).to(dt)
        w = (torch.randn(E, N, K, device=dev) * 0.02).to(dt)
        ours = timed(lambda: ops.scatter2scatter(a, w.permute(0, 2, 1), expert_of_row, rows, out, 1, True, True, offsets))
        dense = timed(lambda: torch.matmul(a, w[0].t(), out=out))
        flops = 2.0 * M * N * K
        points.append({"K": K, "grouped_us_per_round": round(ours / rounds, 2), "library_us_per_round": round(dense / rounds, 2),
                       "grouped_frac_of_bf16_peak": round(flops / (ours * 1e-6) / PEAK_BF16_FLOPS, 4),
                       "library_frac_of_bf16_peak": round(flops / (dense * 1e-6) / PEAK_BF16_FLOPS, 4)})
        del a, w
    ks = np.array([p["K"] for p in points], dtype=np.float64)
    fit = {}
    for who in ("grouped", "library"):
        slope, intercept = np.polyfit(ks, np.array([p[f"{who}_us_per_round"] for p in points]), 1)
        fit[who] = {"us_per_round_outside_the_loop": round(float(intercept), 2),
                    "us_per_round_per_1024_of_reduction": round(float(slope) * 1024, 2),
                    "frac_of_bf16_peak_of_the_loop_alone": round(2.0 * 256 * 256 * 256 * 1024 / (slope * 1024 * 1e-6) / PEAK_BF16_FLOPS, 4)}
    return {"what": f"[{M}, K] x [{N}, K]^T, bf16, {E} experts of {M // E} rows, {rounds:g} rounds of 256 tiles; "
                    "least-squares line through the times per round", "points": points, "fit": fit}


def _aux_hbm_kernels(T: int, H: int, I: int, E: int, k: int) -> list:
    """Stand-alone timings (events on the current stream, outside the timed steps) of the HBM-bound kernels of
    the path at this workload's sizes, plus the histogram / permutation / row moves at fixed large sizes
    (2^20 ids into 256 bins, 2^20 x 4096 bf16 rows; the histogram also at 2^28 ids, which does
    not fit the Infinity Cache)."""

    import torch

    import flash_model_architectures_amd as xma
    from flash_model_architectures_amd import ops

    dev, dt = "cuda", torch.bfloat16
    out = []

    def timed(name, fn, nbytes, iters=10):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        end.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(end) / iters
        out.append(
            {
                "kernel": name,
                "bytes": nbytes,
                "avg_ms": round(ms, 4),
                "gbps": round(nbytes / ms / 1e6, 1),
                "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / PEAK_HBM_BYTES, 4),
            }
        )

    M = T * k
    h = torch.randn(M, 2 * I, device=dev, dtype=dt)
    a = torch.empty(M, I, device=dev, dtype=dt)
    up, gate = h.chunk(2, -1)
    timed(f"swiglu forward [{M}, {I}]", lambda: ops.swiglu_forward_rocm(gate, up, a), 3 * M * I * 2)
    dh = torch.empty_like(h)
    d_up, d_gate = dh.chunk(2, -1)
    timed(f"swiglu backward [{M}, {I}]", lambda: ops.swiglu_backward_rocm(gate, up, a, d_gate, d_up), 5 * M * I * 2)
    del h, a, dh
    for n in (1 << 20, 1 << 28):
        ids = torch.randint(0, 256, (n,), dtype=torch.int32, device=dev)
        counts = torch.empty(256, dtype=torch.uint32, device=dev)
        timed(f"continuous_count 2^{n.bit_length() - 1} int32 ids, 256 bins", lambda: ops.continuous_count_rocm(ids, counts, 256), n * 4 + 1024)
    ids = torch.randint(0, 256, (1 << 20,), dtype=torch.int32, device=dev)
    timed("route_build 2^20 ids, 256 experts (count + offsets + stable permutation)", lambda: xma.route_tokens(ids, 256), 3 * (1 << 20) * 4)
    perm = xma.route_tokens(ids, 256).sorted_scattered_idxs
    rows = torch.empty(1 << 20, 4096, dtype=dt, device=dev).normal_()
    moved = torch.empty_like(rows)
    nbytes = 2 * rows.numel() * 2 + (1 << 20) * 4
    timed("gather rows [2^20, 4096] bf16", lambda: ops.group(rows, perm, moved, None, 1), nbytes, iters=5)
    timed("scatter rows [2^20, 4096] bf16", lambda: ops.ungroup(rows, perm, moved), nbytes, iters=5)
    return out


def main() -> int:
    args = _parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        return 2

    import torch

    import flash_model_architectures_amd as xma
    from flash_model_architectures_amd import _native

    _native.load()  # fail loudly if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    T, H, I = WORKLOAD["tokens"], WORKLOAD["hidden"], WORKLOAD["intermediate"]
    E, k = WORKLOAD["experts"], WORKLOAD["top_k"]
    dt = torch.bfloat16

    if args.only_config is not None:
        workload = OTHER_WORKLOADS[0 if args.only_config == "fine-grained" else 1]
        print(json.dumps({"other_configs": [_other_config(workload, args.other_steps, 2)]}))
        return 0
    if args.reduction_sweep:
        print(json.dumps({"reduction_sweep": _reduction_sweep()}))
        return 0
    if args.library_gemm_only:
        print(json.dumps({"library_gemm": _library_gemms(T, H, I, E, k, iters=max(args.steps, 1))}))
        return 0

    moe = xma.MoE(E, k, H, I, xma.swiglu_packed, True, False, 0.02).to(dt).to(dev)
    x = torch.randn(T, H, device=dev).to(dt).requires_grad_()
    d_y = torch.randn(T, H, device=dev).to(dt)

    def step() -> None:
        y, _ = moe(x)
        y.backward(d_y)
        x.grad = None
        moe.zero_grad(set_to_none=True)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    if args.copy_probe:
        src = torch.empty(1 << 29, dtype=dt, device=dev).normal_()  # 1 GiB read, 1 GiB written
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    timeline = _native.Timeline()
    _native.set_timeline(timeline)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    _native.set_timeline(None)

    ms_per_step = seconds / args.steps * 1e3
    tokens_per_s = T * args.steps / seconds
    gemm_flops = 18.0 * T * k * H * I  # forward 6*M*H*I, backward twice that

    kernels = _kernel_table(timeline.summary(), args.steps)

    dominant = kernels[0]
    if "tflops" in dominant:
        roofline = {
            "kernel": dominant["kernel"],
            "bound": "mfma",
            "achieved": dominant["tflops"],
            "peak": PEAK_BF16_FLOPS / 1e12,
            "unit": "TFLOP/s",
            "frac": dominant["frac_of_bf16_peak"],
            "traffic": _profiled_traffic_bytes().get(dominant["kernel"]),
            "traffic_source": TRAFFIC_PROFILE + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script; "
            "read from that file, not measured in this run)",
            "traffic_profile_blob": _profile_blob_id(),
            "algorithmic_flops_per_launch": dominant["flops_per_launch"],
        }
    else:
        roofline = {
            "kernel": dominant["kernel"],
            "bound": "hbm",
            "achieved": dominant.get("gbps", 0.0),
            "peak": PEAK_HBM_BYTES / 1e9,
            "unit": "GB/s",
            "frac": dominant.get("frac_of_hbm_peak", 0.0),
            "traffic": None,
        }

    gemm_ms = sum(kr["ms_per_step"] for kr in kernels if kr["kernel"].startswith("xma_grouped_gemm"))
    result = {
        "metric": "MoE fwd+bwd tokens/s (Mixtral-shaped bf16 layer, 1 GPU)",
        "value": round(tokens_per_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": WORKLOAD,
        "layer_tflops": round(gemm_flops / (ms_per_step * 1e-3) / 1e12, 2),
        "grouped_gemm_tflops": round(gemm_flops / (gemm_ms * 1e-3) / 1e12, 2) if gemm_ms > 0 else None,
        "grouped_gemm_frac_of_bf16_peak": round(gemm_flops / (gemm_ms * 1e-3) / PEAK_BF16_FLOPS, 4) if gemm_ms else None,
        "roofline": roofline,
        "kernels": kernels,
    }
    if not args.no_other_configs:
        result["other_configs"] = [_other_config(w, args.other_steps, 2) for w in OTHER_WORKLOADS]
    if not args.no_other_dtypes:
        result["other_dtypes"] = [_other_dtype("fp16", 5, 2), _other_dtype("fp32", 2, 1)]
    if not args.no_library_gemm:
        result["library_gemm"] = _library_gemms(T, H, I, E, k)
    if not args.no_aux:
        result["aux_hbm_kernels"] = _aux_hbm_kernels(T, H, I, E, k)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = _cpu_baseline(moe, x, d_y, args.cpu_sample_tokens)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
