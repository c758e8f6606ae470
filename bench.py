"""Benchmark of the gated delta-rule path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload 1|2|4] [--no-cpu-baseline] [--no-decode]
                    [--no-other-configs]

A "step" is one chunked forward (``chunk_gated_delta_rule``) over one batch of synthetic input of
the benchmark configuration (default: configuration 1, B=4, T=4096, H=16, K=V=128, bf16, chunk 64),
inputs already resident in HBM.  Prints ONE JSON line:

  value        tokens/s of the whole step (B*T / wall time per step, all kernels and the allocation of the
               outputs included; the operator keeps its workspace between steps)
  roofline     the dominant kernel of the step against the bf16 dense MFMA peak: algorithmic
               FLOPs of the contractions that kernel performs / its HIP-event duration
  decode       the decode step (configuration 3: 256 sequences x 32 heads, fp32 state 512 MiB
               updated in place) against the HBM peak, state buffers rotated so the state
               cannot live in the 256 MB Infinity Cache
  conv         the depthwise causal convolution in front of the operator, same batch, against the HBM peak
  epilogue     rmsnorm(o * silu(gate)) behind the operator, same batch, against the HBM peak
  cpu_baseline the naive token-by-token torch restatement of the operator (oracle/), timed on
               this host's cores on a bounded prefix of the same workload
  backward     one backward of the operator at the headline shape (and, under `other`, at the shipped head shape)
  forward_other the same forward with prepare and scan as two kernels (the headline configuration runs them as one
               launch by default), on configurations 2 (packed sequences) and 4 (long context, V=256; both ways), and
               on the head shape of the reference's shipped configurations (B=8, T=4096, H=2, K=256, V=512)
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from dataclasses import replace


ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E

# HBM bytes per launch are not measurable from inside this process: they are rocprofv3 --pmc readings of
# FETCH_SIZE and WRITE_SIZE (KiB per dispatch) for this very command, each scaled by what the same counter reads
# for a plain 1 GiB copy.  The readings live in profiles/hbm_traffic_counters.json together with a digest of the
# kernel sources they were taken on; with other sources (a kernel was changed since) every traffic figure is null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_counters.json")
_LAUNCH_MODE = []  # keeps the kernel-flag context of --two-kernels alive
_traffic_table = None


def kernel_sources_digest() -> str:
    """sha256 over the HIP sources and headers the library is built from, in name order."""
    import hashlib

    digest = hashlib.sha256()
    csrc = os.path.join(ROOT, "lm_engine_amd", "csrc")
    names = sorted(n for n in os.listdir(csrc) if n.endswith((".hip", ".h")))
    for path in [os.path.join(csrc, n) for n in names] + [os.path.join(ROOT, "include", "gdn_hip.h")]:
        with open(path, "rb") as f:
            digest.update(os.path.basename(path).encode() + b"\0" + f.read())
    return digest.hexdigest()


def measured_traffic(workload: str, kernel: str):
    """HBM bytes one launch of ``kernel`` moves on ``workload`` (counter readings, see above), or None."""
    global _traffic_table
    if _traffic_table is None:
        _traffic_table = {}
        try:
            with open(TRAFFIC_FILE) as f:
                table = json.load(f)
            if table.get("sources_sha256") == kernel_sources_digest():
                _traffic_table = table
        except (OSError, ValueError):
            pass
    entry = _traffic_table.get("kernels", {}).get(f"{workload}/{kernel}")
    if entry is None:
        return None
    kib = entry["fetch_size_kib"] * _traffic_table["fetch_size_scale"] + entry["write_size_kib"] * _traffic_table["write_size_scale"]
    return int(kib * 1024)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", type=int, default=1, choices=(1, 2, 4))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true", help="skip the decode, convolution, epilogue and backward legs")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target duration of the CPU baseline sample")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the forward legs of configurations 2 and 4")
    ap.add_argument("--two-kernels", action="store_true",
                    help="run the headline step and everything after it with prepare and scan as two kernels "
                         "(Kernel.gated_delta_rule_fused_launch off) also where the library would use one launch")
    ap.add_argument("--cycle-budget", action="store_true",
                    help="instead of the benchmark: run the headline forward (as two kernels) on the measurement build of the "
                         "library (python -m lm_engine_amd.build --cycle-budget) and print the shader-clock cycles a compute "
                         "wave of the half-slice scan spends in each group of MFMAs of its chunk loop, then one backward at the "
                         "headline shape and one at the shipped head shape and the cycles of the chunk-local backward "
                         "kernel's steps")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy, the known-size kernel the HBM counters are scaled by")
    return ap.parse_args()


DEVICE_WARMUP_MS = 60.0


def device_warmup(call, ms: float = DEVICE_WARMUP_MS):
    """Runs ``call`` back to back, untimed, for about ``ms`` of wall time.  An idle MI355X sits at low clocks and needs
    some 20 ms of sustained work to reach the clocks it then holds: a leg that starts timing after a handful of warm-up
    steps measures the ramp (configuration 1: 0.132 ms per step over the first 7 ms, 0.114 over the next 6, then 0.107
    for as long as the loop runs).  Every leg therefore first brings the device to that state with its own step; the
    W warm-up steps and the K timed steps follow immediately."""
    import torch

    takes_index = call.__code__.co_argcount == 1  # the decode leg rotates its state buffers
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n = 0
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(8):
            call(n) if takes_index else call()
            n += 1
        if n % 64 == 0:  # keep the launch queue short so that the wall clock above means device time
            torch.cuda.synchronize()
    torch.cuda.synchronize()


def launch_mode(two_kernels: bool):
    """Context of a leg: the library's default (prepare and scan in one launch for the shapes where that is faster), or
    prepare and scan as two kernels whatever the shape."""
    import contextlib

    from lm_engine_amd.kernels import Kernel, enable_kernels

    return enable_kernels([Kernel.gated_delta_rule], reset=True) if two_kernels else contextlib.nullcontext()


def chunk_forward_leg(w, steps, warmup, two_kernels):
    """Wall time per forward of workload ``w`` and the HIP-event durations of its kernels, one launch mode."""
    import torch

    import lm_engine_amd
    from lm_engine_amd.ops import chunk_forward_kernel_times, fused_launch_applies
    from lm_engine_amd.workloads import chunk_fwd_flops_per_token_head, make_inputs

    inp = make_inputs(w, device="cuda")
    with launch_mode(two_kernels):
        one_launch = fused_launch_applies(inp["q"], inp["v"], inp["cu_seqlens"])
        device_warmup(lambda: lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True))
        for _ in range(warmup):
            lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / steps * 1e3
        sums: dict[str, float] = {}
        for _ in range(steps):
            for name, t in chunk_forward_kernel_times(**inp, output_final_state=True).items():
                sums[name] = sums.get(name, 0.0) + t
    n_seq = w.B if inp["cu_seqlens"] is None else inp["cu_seqlens"].numel() - 1
    tflops = w.B * w.T * w.H * chunk_fwd_flops_per_token_head(w.K, w.V)["dense"] / (ms * 1e-3) / 1e12
    del inp
    torch.cuda.empty_cache()
    return {
        "workload": w.name, "B": w.B, "T": w.T, "H": w.H, "K": w.K, "V": w.V, "sequences": n_seq,
        "launch": "prepare and scan in one launch" if one_launch else "prepare, then scan",
        "ms_per_step": round(ms, 4),
        "tokens_per_s": round(w.B * w.T / (ms * 1e-3), 1),
        "tflops_dense": round(tflops, 1),
        "mfma_frac_dense": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
        # (in the one-launch mode the whole launch is booked under chunk_scan)
        "kernel_ms": {name: round(total / steps, 4) for name, total in sums.items()},
    }  # fmt: skip


def bench_chunk(w, steps, warmup, two_kernels=False):
    import torch

    import lm_engine_amd
    from lm_engine_amd.ops import chunk_forward_kernel_times, fused_launch_applies
    from lm_engine_amd.workloads import chunk_fwd_bytes_per_token_head, chunk_fwd_flops_per_token_head, make_inputs

    if two_kernels:  # for the rest of the run
        _LAUNCH_MODE.append(launch_mode(True))
        _LAUNCH_MODE[-1].__enter__()
    inp = make_inputs(w, device="cuda")
    fused_launch = fused_launch_applies(inp["q"], inp["v"], inp["cu_seqlens"])
    call = lambda: lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)  # noqa: E731

    device_warmup(call)
    for _ in range(warmup):
        call()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        call()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / steps * 1e3

    # per-kernel durations: HIP events recorded on the launch stream around every kernel of the step
    sums: dict[str, float] = {}
    for _ in range(steps):
        for name, ms in chunk_forward_kernel_times(**inp, output_final_state=True).items():
            sums[name] = sums.get(name, 0.0) + ms
    kernel_ms = {name: total / steps for name, total in sums.items()}

    tokens = w.B * w.T
    token_heads = tokens * w.H
    flops = chunk_fwd_flops_per_token_head(w.K, w.V)
    n_seq = w.B if inp["cu_seqlens"] is None else inp["cu_seqlens"].numel() - 1
    state_bytes = n_seq * w.H * w.K * w.V * 4 * (2 if inp["initial_state"] is not None else 1)
    algo_bytes = token_heads * chunk_fwd_bytes_per_token_head(w.K, w.V) + state_bytes

    per_kernel = {}
    for name, part in (("chunk_prepare", "prepare"), ("chunk_scan", "scan")):
        if fused_launch:  # one launch does both parts; it is booked under chunk_scan
            if name == "chunk_prepare":
                continue
            part = "dense"
        tflops = token_heads * flops[part] / (kernel_ms[name] * 1e-3) / 1e12
        key = "chunk_fused" if fused_launch else name
        per_kernel[key] = {"ms": round(kernel_ms[name], 4), "algorithmic_flop_per_token_head": flops[part],
                           "tflops": round(tflops, 1), "mfma_frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
                           "traffic": measured_traffic(w.name, key)}  # fmt: skip
    dominant = max(per_kernel, key=lambda name: per_kernel[name]["ms"])
    # HBM bytes of the whole step (every kernel of it), or null when a kernel has no reading
    step_traffic = [k["traffic"] for k in per_kernel.values()]
    step_traffic = None if any(t is None for t in step_traffic) else sum(step_traffic)
    whole_tflops = token_heads * flops["dense"] / (ms_per_step * 1e-3) / 1e12

    result = {
        "metric": "GDN chunk-fwd tokens/s",
        "value": round(tokens / (ms_per_step * 1e-3), 1),
        "unit": "tokens/s",
        "ms_per_step": round(ms_per_step, 4),
        "dtype": "bf16",
        "config": {"workload": w.name, "B": w.B, "T": w.T, "H": w.H, "K": w.K, "V": w.V, "chunk": 64,
                   "sequences": n_seq, "initial_state": inp["initial_state"] is not None,
                   "launch": "prepare and scan in one launch" if fused_launch else "prepare, then scan"},  # fmt: skip
        "roofline": {
            "kernel": dominant,
            "bound": "mfma",
            "achieved": per_kernel[dominant]["tflops"],
            "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": per_kernel[dominant]["mfma_frac"],
            "traffic": step_traffic,
            "traffic_scope": "whole step: " + " + ".join(per_kernel) + " (per kernel under step.kernels)",
            "algorithmic_bytes": int(algo_bytes),
            # the same step against the other roof: its algorithmic bytes over the sum of its kernels' durations
            "hbm": {
                "achieved": round(algo_bytes / (sum(k["ms"] for k in per_kernel.values()) * 1e-3) / 1e9, 1),
                "peak": HBM_PEAK_GBS,
                "unit": "GB/s",
                "frac": round(algo_bytes / (sum(k["ms"] for k in per_kernel.values()) * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            },
        },
        "step": {
            "tflops_dense": round(whole_tflops, 1),
            "mfma_frac_dense": round(whole_tflops / MFMA_BF16_PEAK_TFLOPS, 4),
            "tflops_strict": round(token_heads * flops["strict"] / (ms_per_step * 1e-3) / 1e12, 1),
            "tflops_wy_count": round(token_heads * flops["wy"] / (ms_per_step * 1e-3) / 1e12, 1),
            "algorithmic_gbs": round(algo_bytes / (ms_per_step * 1e-3) / 1e9, 1),
            "hbm_frac": round(algo_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "kernels": per_kernel,
        },
    }
    return result, inp


def bench_decode(steps, warmup):
    import torch

    import lm_engine_amd
    from lm_engine_amd.workloads import decode_bytes_per_seq_head, get_workload, make_inputs

    w = get_workload(3)
    inp = make_inputs(w, device="cuda")
    states = [inp["initial_state"].clone() for _ in range(3)]  # 3 x 512 MiB > Infinity Cache

    def call(i):
        args = dict(inp, initial_state=states[i % len(states)])
        return lm_engine_amd.fused_recurrent_gated_delta_rule(**args, output_final_state=True, inplace_state=True)

    device_warmup(call)
    for i in range(warmup):
        call(i)
    torch.cuda.synchronize()
    # one pair of events around all the launches: a pair per launch adds its own handling (~5 us) to every bracket
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        call(i)
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) / steps * 1e3
    kernel_ms = start.elapsed_time(stop) / steps
    nbytes = decode_bytes_per_seq_head(w.K, w.V) * w.B * w.H
    gbs = nbytes / (kernel_ms * 1e-3) / 1e9
    return {
        "workload": w.name,
        "sequences": w.B, "H": w.H, "K": w.K, "V": w.V,
        "ms_per_step": round(wall_ms, 4),
        "kernel_ms": round(kernel_ms, 4),
        "seq_tokens_per_s": round(w.B / (wall_ms * 1e-3), 1),
        "roofline": {"kernel": "recurrent_kernel", "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic("cfg3_decode_bf16", "recurrent_kernel")},
    }  # fmt: skip


def bench_conv(w, steps, warmup):
    """The depthwise causal convolution (kernel size 4, bias, SiLU) over the fused q | k | v projection of
    the same workload: [B, T, H (2K + V)] bf16 in, same shape out, carried state written.  HBM-bound:
    algorithmic bytes = one read of x + one write of y."""
    import torch

    import lm_engine_amd

    C = w.H * (2 * w.K + w.V)
    gen = torch.Generator("cpu").manual_seed(4321)
    x = torch.randn(w.B, w.T, C, generator=gen).to(torch.bfloat16).cuda()
    weight = (0.5 * torch.randn(C, 1, 4, generator=gen)).to(torch.bfloat16).cuda()
    bias = (0.1 * torch.randn(C, generator=gen)).to(torch.bfloat16).cuda()
    call = lambda: lm_engine_amd.depthwise_causal_convolution(x, weight, bias, None, None, True, "silu")  # noqa: E731
    device_warmup(call)
    for _ in range(warmup):
        call()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        call()
    stop.record()
    torch.cuda.synchronize()
    kernel_ms = start.elapsed_time(stop) / steps  # back-to-back launches, one pair of events around all of them
    nbytes = 2 * x.numel() * x.element_size()
    gbs = nbytes / (kernel_ms * 1e-3) / 1e9
    return {
        "workload": f"conv1d_k4_silu_bf16 B={w.B} S={w.T} C={C}",
        "kernel_ms": round(kernel_ms, 4),
        "tokens_per_s": round(w.B * w.T / (kernel_ms * 1e-3), 1),
        "roofline": {"kernel": "causal_conv1d_kernel", "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(w.name, "causal_conv1d_kernel")},
    }  # fmt: skip


def bench_epilogue(w, steps, warmup):
    """rmsnorm(o * silu(gate)) * weight over the operator's output of the same workload, gate read as a
    slice of a wider projection.  HBM-bound: algorithmic bytes = o and gate in, y out."""
    import torch

    import lm_engine_amd

    gen = torch.Generator("cpu").manual_seed(987)
    o = torch.randn(w.B, w.T, w.H, w.V, generator=gen).to(torch.bfloat16).cuda()
    proj = torch.randn(w.B, w.T, 2 * w.H + w.H * w.V, generator=gen).to(torch.bfloat16).cuda()
    gate = proj[..., 2 * w.H:]
    weight = torch.ones(w.V, dtype=torch.bfloat16, device="cuda")
    call = lambda: lm_engine_amd.gated_rmsnorm(o, gate, weight, 1e-5)  # noqa: E731
    device_warmup(call)
    for _ in range(warmup):
        call()
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for start, stop in events:
        start.record()
        call()
        stop.record()
    torch.cuda.synchronize()
    kernel_ms = sum(start.elapsed_time(stop) for start, stop in events) / steps
    nbytes = 3 * o.numel() * o.element_size()
    gbs = nbytes / (kernel_ms * 1e-3) / 1e9
    return {
        "workload": f"gated_rmsnorm_bf16 B={w.B} T={w.T} H={w.H} V={w.V}",
        "kernel_ms": round(kernel_ms, 4),
        "roofline": {"kernel": "gated_rmsnorm_kernel", "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(w.name, "gated_rmsnorm_kernel")},
    }  # fmt: skip


def cpu_baseline(w, inp_gpu, target_seconds):
    """Naive recurrent torch restatement on this host's cores, on a bounded sample of the workload:
    whole sequences in order (all heads) until the time budget is used, or a prefix of the first
    sequence if even that does not fit (the cost is exactly linear in the token count)."""
    import torch

    from oracle import recurrent_gated_delta_rule_ref
    from oracle.c_oracle import recurrent_gated_delta_rule_c

    cores = torch.get_num_threads()
    cpu = {n: (x.cpu() if isinstance(x, torch.Tensor) else x) for n, x in inp_gpu.items()}
    packed = cpu["cu_seqlens"] is not None
    bounds = [int(x) for x in cpu["cu_seqlens"]] if packed else None
    n_seq = len(bounds) - 1 if packed else w.B

    def sequence(i, tokens=None):
        if packed:
            t0, t1 = bounds[i], bounds[i + 1] if tokens is None else bounds[i] + tokens
            sub = {n: cpu[n][:, t0:t1] for n in ("q", "k", "v", "g", "beta") if cpu[n] is not None}
        else:
            t1 = w.T if tokens is None else tokens
            sub = {n: cpu[n][i : i + 1, :t1] for n in ("q", "k", "v", "g", "beta") if cpu[n] is not None}
        h0 = cpu["initial_state"]
        return dict(sub, initial_state=None if h0 is None else h0[i : i + 1], scale=cpu["scale"])

    first_len = (bounds[1] - bounds[0]) if packed else w.T
    probe = min(64, first_len)
    t0 = time.perf_counter()
    recurrent_gated_delta_rule_ref(**sequence(0, probe), output_final_state=True)
    per_token = (time.perf_counter() - t0) / probe

    tokens, seconds, what = 0, 0.0, ""
    if per_token * first_len > target_seconds:
        tokens = max(probe, int(target_seconds / per_token))
        t0 = time.perf_counter()
        recurrent_gated_delta_rule_ref(**sequence(0, tokens), output_final_state=True)
        seconds = time.perf_counter() - t0
        what = f"first {tokens} of {first_len} tokens of the first sequence"
    else:
        done = 0
        while done < n_seq and seconds < target_seconds:
            inp = sequence(done)
            t0 = time.perf_counter()
            recurrent_gated_delta_rule_ref(**inp, output_final_state=True)
            seconds += time.perf_counter() - t0
            tokens += inp["q"].size(1)
            done += 1
        what = f"{done} of {n_seq} whole sequences ({tokens} tokens)"

    full = sequence(0)
    t0 = time.perf_counter()
    recurrent_gated_delta_rule_c(**full, output_final_state=True, f64_state=False)
    c_seconds = time.perf_counter() - t0

    return {
        "value": round(tokens / seconds, 1),
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{w.name}: {what}, all {w.H} heads, fp32 torch token loop, {seconds:.1f} s",
        "c_port_tokens_per_s": round(first_len / c_seconds, 1),
        "c_port_sample": f"first sequence ({first_len} tokens), C restatement with OpenMP over heads, {c_seconds:.2f} s",
    }


def cycle_budget(w):
    """The chunk loop of the half-slice scan, group by group, in shader-clock cycles per chunk: the forward of workload
    ``w`` as two kernels on ``libgdn_hip_cycles.so``, whose scan reads the clock between its groups of MFMAs (wave 0 of
    every 16th workgroup reports).  The instrumented loop is a few hundred cycles per chunk slower than the real one
    (each reading waits for the wave's LDS reads in flight); the kernel's event time in the same build is printed with
    it, next to the uninstrumented figure of the bench line."""
    import ctypes

    import torch

    import lm_engine_amd
    from lm_engine_amd import _lib
    from lm_engine_amd.build import CYCLE_BUDGET_LIBRARY_PATH
    from lm_engine_amd.ops import chunk_forward_kernel_times
    from lm_engine_amd.workloads import make_inputs

    if not os.path.exists(CYCLE_BUDGET_LIBRARY_PATH):
        raise SystemExit(f"{CYCLE_BUDGET_LIBRARY_PATH} is missing: python -m lm_engine_amd.build --cycle-budget")
    _lib.LIBRARY_PATH = CYCLE_BUDGET_LIBRARY_PATH  # before the first load
    lib = _lib.load_library()
    lib.gdn_cycle_budget_read.argtypes = [ctypes.POINTER(ctypes.c_uint64), ctypes.c_int]
    lib.gdn_cycle_budget_read.restype = ctypes.c_int
    inp = make_inputs(w, device="cuda")
    names = ("k_s0", "s0t_qt", "t_x", "kt_vnew", "vnewt_pt", "between_chunks")
    with launch_mode(True):
        call = lambda: lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)  # noqa: E731
        device_warmup(call)
        times = [chunk_forward_kernel_times(**inp, output_final_state=True) for _ in range(10)]
        call()
        slots = 16
        out = (ctypes.c_uint64 * (slots * 8))()
        _lib.check_status(lib.gdn_cycle_budget_read(out, slots), "gdn_cycle_budget_read")
    rows = [[out[8 * i + j] for j in range(7)] for i in range(slots)]
    rows = [r for r in rows if r[6] > 0]
    per_chunk = {n: round(sum(r[j] / r[6] for r in rows) / len(rows), 1) for j, n in enumerate(names)}
    scan_ms = sum(t["chunk_scan"] for t in times) / len(times)
    chunks = rows[0][6]
    return {
        "workload": w.name, "kernel": "chunk_scan32_kernel, half-slice compute wave 0", "sampled_workgroups": len(rows),
        "chunks_per_chain": int(chunks), "cycles_per_chunk": per_chunk, "cycles_per_chunk_total": round(sum(per_chunk.values()), 1),
        "scan_kernel_ms_instrumented": round(scan_ms, 4),
        "implied_shader_clock_ghz": round(sum(per_chunk.values()) * chunks / (scan_ms * 1e6), 3),
    }  # fmt: skip


def calibrate_copy():
    """A plain device-to-device copy of 1 GiB: the kernel of known traffic (1 GiB read, 1 GiB written)
    against which FETCH_SIZE / WRITE_SIZE readings of the other kernels are scaled."""
    import torch

    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()


def bench_layer_backward_kernels(w, steps, warmup):
    """The backward kernels of the convolution and of the gated norm on the shapes of ``bench_conv`` and
    ``bench_epilogue``.  HBM-bound: algorithmic bytes = x and dy in, dx out (convolution); o, gate and dy in, d_o and
    d_gate out (norm).  One pair of events around back-to-back launches, the partial sums' reduction included."""
    import torch

    from lm_engine_amd.conv import _convolution_backward
    from lm_engine_amd.layer_ops import _gated_rmsnorm_backward

    def timed(call):
        device_warmup(call)
        for _ in range(warmup):
            call()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(steps):
            call()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / steps

    gen = torch.Generator("cpu").manual_seed(4322)
    C = w.H * (2 * w.K + w.V)
    x = torch.randn(w.B, w.T, C, generator=gen).to(torch.bfloat16).cuda()
    dy = torch.randn(w.B, w.T, C, generator=gen).to(torch.bfloat16).cuda()
    weight = (0.5 * torch.randn(C, 1, 4, generator=gen)).to(torch.bfloat16).cuda()
    bias = (0.1 * torch.randn(C, generator=gen)).to(torch.bfloat16).cuda()
    conv_ms = timed(lambda: _convolution_backward(x, weight, bias, None, None, dy, "silu"))
    conv_gbs = 3 * x.numel() * 2 / (conv_ms * 1e-3) / 1e9

    o = torch.randn(w.B, w.T, w.H, w.V, generator=gen).to(torch.bfloat16).cuda()
    proj = torch.randn(w.B, w.T, 2 * w.H + w.H * w.V, generator=gen).to(torch.bfloat16).cuda()
    gate = proj[..., 2 * w.H:]
    do = torch.randn(w.B, w.T, w.H, w.V, generator=gen).to(torch.bfloat16).cuda()
    nweight = torch.ones(w.V, dtype=torch.bfloat16, device="cuda")
    norm_ms = timed(lambda: _gated_rmsnorm_backward(o, gate, nweight, 1e-5, do))
    norm_gbs = 5 * o.numel() * 2 / (norm_ms * 1e-3) / 1e9
    return {
        "conv": {"workload": f"conv1d_k4_silu_bf16 backward B={w.B} S={w.T} C={C}", "ms": round(conv_ms, 4),
                 "roofline": {"kernel": "causal_conv1d_bwd_kernel", "bound": "hbm", "achieved": round(conv_gbs, 1),
                              "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(conv_gbs / HBM_PEAK_GBS, 4), "traffic": None}},
        "norm": {"workload": f"gated_rmsnorm_bf16 backward B={w.B} T={w.T} H={w.H} V={w.V}", "ms": round(norm_ms, 4),
                 "roofline": {"kernel": "gated_rmsnorm_bwd_kernel", "bound": "hbm", "achieved": round(norm_gbs, 1),
                              "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(norm_gbs / HBM_PEAK_GBS, 4), "traffic": None}},
    }  # fmt: skip


LOCAL_GROUPS = ("stage_slab", "barrier_a", "row_sums", "ask_ds1", "ask_next_slab", "products_s0", "barrier_b",
                "stage_ds1", "barrier_c", "products_ds1", "barrier_d", "reduce_dot", "phase2", "phase3", "stores_tail")


def cycle_budget_backward_local(w):
    """The chunk-local backward kernel (``gdn_chunk_bwd_local``) step by step, in shader-clock cycles per chunk: one
    backward of workload ``w`` on ``libgdn_hip_cycles.so`` (loaded by ``cycle_budget`` before this), whose kernel reads
    the clock between its steps (wave 0 of 32 workgroups spread over the grid reports).  Phase 1 runs once per slab of 64
    value columns: its groups are sums over the slabs of a chunk."""
    import ctypes

    import torch

    from lm_engine_amd import _lib
    from lm_engine_amd.backward import gated_delta_rule_backward
    from lm_engine_amd.workloads import make_inputs

    lib = _lib.load_library()
    inp = make_inputs(w, device="cuda")
    do = torch.randn(inp["v"].shape, generator=torch.Generator("cpu").manual_seed(555)).to(inp["v"].dtype).cuda()
    call = lambda: gated_delta_rule_backward(  # noqa: E731
        inp["q"], inp["k"], inp["v"], inp["g"], inp["beta"], do, None, scale=inp["scale"],
        initial_state=inp["initial_state"], cu_seqlens=inp["cu_seqlens"])  # fmt: skip
    device_warmup(call)
    call()
    out = (ctypes.c_uint64 * 512)()
    _lib.check_status(lib.gdn_cycle_budget_read(out, 64), "gdn_cycle_budget_read")
    rows = [[out[16 * i + j] for j in range(16)] for i in range(32)]
    rows = [r for r in rows if r[15] > 0]
    per_chunk = {n: round(sum(r[j] for r in rows) / len(rows), 1) for j, n in enumerate(LOCAL_GROUPS)}
    return {
        "workload": w.name, "K": w.K, "V": w.V, "kernel": "chunk_local_grads_kernel, wave 0", "sampled_workgroups": len(rows),
        "slabs_per_chunk": int(rows[0][15]), "cycles_per_chunk": per_chunk, "cycles_per_chunk_total": round(sum(per_chunk.values()), 1),
    }  # fmt: skip


def bench_backward(w, inp, steps, warmup):
    """One backward pass of the chunked operator on the same workload (``lm_engine_amd.backward``), gradient
    of the output only.  Wall time per call with the device idle before and after."""
    import torch

    from lm_engine_amd.backward import gated_delta_rule_backward
    from lm_engine_amd.ops import backward_kernels_apply

    gen = torch.Generator("cpu").manual_seed(555)
    do = torch.randn(inp["v"].shape, generator=gen).to(inp["v"].dtype).cuda()
    call = lambda: gated_delta_rule_backward(  # noqa: E731
        inp["q"], inp["k"], inp["v"], inp["g"], inp["beta"], do, None, scale=inp["scale"],
        initial_state=inp["initial_state"], cu_seqlens=inp["cu_seqlens"])  # fmt: skip
    steps, warmup = max(1, min(steps, 5)), max(1, min(warmup, 2))
    device_warmup(call)
    for _ in range(warmup):
        call()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        call()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    return {
        "workload": w.name,
        "steps": steps,
        "ms_per_backward": round(ms, 3),
        "tokens_per_s": round(inp["q"].size(0) * inp["q"].size(1) / (ms * 1e-3), 1),
        "composition": ("5 kernel launches (and the 7 us chunk-offsets helper): backward prepare, forward prepare + saving scan (forward sweep), saving scan "
                        "over the mirror problem with every row scanned over its own chunks (reverse sweep), chunk-local "
                        "gradients; chunk states, V~ and Y pass between them as bf16"
                        if backward_kernels_apply(w.K, w.V) and inp["cu_seqlens"] is not None else
                        "4 kernel launches: backward prepare (also writes the forward sweep's records), saving scan "
                        "on those records (forward sweep), saving scan over the mirror problem (reverse sweep), "
                        "chunk-local gradients; chunk states, V~ and Y pass between them as bf16"
                        if backward_kernels_apply(w.K, w.V) else
                        "2 saving scans + rocBLAS batched GEMMs + elementwise torch ops"),
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this build has no multi-GPU path (got --gpus {args.gpus}). "
              "The operator shards over sequences and heads without any exchange; run one process per GPU.",
              file=sys.stderr)  # fmt: skip
        sys.exit(2)

    import torch

    from lm_engine_amd.workloads import get_workload

    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the gated delta rule has no CPU path", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)

    if args.cycle_budget:
        print(json.dumps({"cycle_budget": cycle_budget(get_workload(args.workload))}))
        shipped = replace(get_workload(1, B=8, H=2, K=256, V=512), name="shipped_head_shape_k256_v512_bf16")
        print(json.dumps({"cycle_budget_backward_local": [cycle_budget_backward_local(get_workload(args.workload)),
                                                          cycle_budget_backward_local(shipped)]}))
        return
    w = get_workload(args.workload)
    result, inp = bench_chunk(w, args.steps, args.warmup, args.two_kernels)
    decode = None if args.no_decode else bench_decode(args.steps, args.warmup)
    conv = None if args.no_decode else bench_conv(w, args.steps, args.warmup)
    epilogue = None if args.no_decode else bench_epilogue(w, args.steps, args.warmup)
    backward = None if args.no_decode else bench_backward(w, inp, args.steps, args.warmup)
    if backward is not None:
        backward["layer_kernels"] = bench_layer_backward_kernels(w, args.steps, args.warmup)
        if not args.no_other_configs:
            # the same leg at the head shape of the reference's shipped configurations (K = 256, V = 512)
            import torch

            from lm_engine_amd.workloads import make_inputs

            shipped = replace(get_workload(1, B=8, H=2, K=256, V=512), name="shipped_head_shape_k256_v512_bf16")
            backward["other"] = [bench_backward(shipped, make_inputs(shipped, device="cuda"), args.steps, args.warmup)]
            torch.cuda.empty_cache()
            # and on the packed, ragged batch of configuration 2 (the rows of its mirror problem are scanned over their own lengths)
            ragged = get_workload(2)
            backward["other"].append(bench_backward(ragged, make_inputs(ragged, device="cuda"), args.steps, args.warmup))
            torch.cuda.empty_cache()
    other = None
    if not args.no_other_configs:
        # the forward on the other chunked configurations, and with prepare and scan in one launch where that qualifies
        other = [chunk_forward_leg(w, args.steps, args.warmup, two_kernels=True)]
        for index in (2, 4):
            if index != args.workload:
                other.append(chunk_forward_leg(get_workload(index), args.steps, args.warmup, two_kernels=False))
        # the head shape of the reference's shipped configurations (k_head_dim 256, v_head_dim 512, 2 heads, micro-batch 8)
        shipped = get_workload(1, B=8, H=2, K=256, V=512)
        other.append(chunk_forward_leg(replace(shipped, name="shipped_head_shape_k256_v512_bf16"), args.steps, args.warmup, two_kernels=False))
    baseline = None if args.no_cpu_baseline else cpu_baseline(w, inp, args.cpu_seconds)
    if args.calibrate_copy:
        calibrate_copy()

    line = {
        "metric": result["metric"],
        "value": result["value"],
        "unit": result["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": result["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": result["dtype"],
        "data": "synthetic",
        "config": result["config"],
        "roofline": result["roofline"],
        "cpu_baseline": baseline,
        "step": result["step"],
        "decode": decode,
        "conv": conv,
        "epilogue": epilogue,
        "backward": backward,
        "forward_other": other,
        "device": torch.cuda.get_device_name(0),
        "device_warmup": (f"every leg first runs its own step back to back, untimed, for {DEVICE_WARMUP_MS:.0f} ms of wall time "
                          "(an idle device needs ~20 ms of sustained work to reach the clocks it then holds), then its warm-up "
                          "steps, then the timed steps"),
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
