#!/usr/bin/env python3
"""Benchmark of the hot path: causal flash-attention forward + backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config nstar|c1|c2|c3|c4|c5]

A step is one forward + one backward pass of attention over one synthetic batch that is already resident
in HBM.  The default workload is the target shape of the baseline (B=4, H=32, T=4096, d=128, bf16, causal);
the five baseline configurations are timed briefly as well and reported under "configs".  One JSON line is
printed.  FLOPs are the algorithmic ones of the baseline's work model: 2 (forward) + 5 (backward) matrix
products of 2*T^2*d per (batch, query head), halved for the causal mask, i.e. 7*B*H*T^2*d in total;
recomputation inside the two-kernel backward is not counted.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2516.6, "fp16": 2516.6, "fp32": 157.3}  # MI355X dense MFMA (256 CU x 2.4 GHz)
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E

# name: (B, Hq, Hkv, T, d, dtype, sigma_qk, description)
CONFIGS = {
    "c1": (4, 4, 4, 48, 16, "fp32", 1.0, "tiny quickstart LM attention B4 H4 T48 d16 fp32"),
    "c2": (8, 12, 12, 1024, 64, "bf16", 0.70710678, "GPT-2-small-shaped B8 H12 T1024 d64 bf16"),
    "c3": (4, 32, 32, 2048, 128, "bf16", 1.0, "Llama-7B-shaped B4 H32 T2048 d128 bf16"),
    "c4": (4, 32, 8, 4096, 128, "bf16", 1.0, "GQA B4 Hq32/Hkv8 T4096 d128 bf16"),
    "c5": (1, 16, 16, 16384, 64, "fp16", 3.0, "long-context B1 H16 T16384 d64 fp16"),
    "nstar": (4, 32, 32, 4096, 128, "bf16", 1.0, "target shape B4 H32 T4096 d128 bf16 causal"),
}
SEEDS = {"c1": 1, "c2": 2, "c3": 3, "c4": 4, "c5": 5, "nstar": 6}
# algorithmic matrix products per kernel (units of B*H*T^2*d FLOPs, causal-halved)
KERNEL_UNITS = {"fwd_mfma": 2.0, "dkdv_mfma": 4.0, "dq_mfma": 1.0, "fwd_f32": 2.0, "dkdv_f32": 4.0, "dq_f32": 1.0}
# kernel names as timed by the library -> the kernel functions they stand for in the profiler's tables
PROFILED_KERNELS = {"fwd_mfma": ("fwd_mfma_kernel",), "dkdv_mfma": ("dkdv_split_kernel", "dkdv_mfma_kernel"),
                    "dq_mfma": ("dq_mfma_kernel",)}
COUNTER_SUMMARIES = {"nstar": "nstar_b4_h32_t4096_d128_bf16_counters.txt"}


def measured_traffic_bytes(config, kernel):
    """HBM bytes per launch of `kernel` as measured with rocprofv3 (FETCH_SIZE and WRITE_SIZE runs, scaled by a plain
    copy kernel of known size): the total_MiB column of the committed counter summary of this workload, or None."""
    name = COUNTER_SUMMARIES.get(config)
    if name is None or kernel not in PROFILED_KERNELS:
        return None
    try:
        lines = open(os.path.join(ROOT, "profiles", name)).read().splitlines()
    except OSError:
        return None
    column = None
    for line in lines:
        fields = line.split()
        if "total_MiB" in fields and "FETCH_SIZE" in fields:
            column = len(fields) - fields.index("total_MiB")  # counted from the right: kernel names hold spaces
            continue
        if column is not None and line.startswith(PROFILED_KERNELS[kernel]):
            try:
                return float(fields[-column]) * 2 ** 20
            except (ValueError, IndexError):
                return None
    return None


def make_inputs(torch, name):
    b, hq, hkv, t, d, dtype, sigma, _ = CONFIGS[name]
    tdt = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}[dtype]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5E17 + SEEDS[name])
    q = (sigma * torch.randn(b, hq, t, d, device="cuda", generator=gen)).to(tdt)
    k = (sigma * torch.randn(b, hkv, t, d, device="cuda", generator=gen)).to(tdt)
    v = torch.randn(b, hkv, t, d, device="cuda", generator=gen).to(tdt)
    g = torch.randn(b, hq, t, d, device="cuda", generator=gen).to(tdt)
    return q, k, v, g


class Workload:
    def __init__(self, torch, name):
        import sentinel_amd
        self.torch = torch
        self.fa = sentinel_amd
        self.name = name
        self.b, self.hq, self.hkv, self.t, self.d, self.dtype, _, self.desc = CONFIGS[name]
        self.q, self.k, self.v, self.g = make_inputs(torch, name)
        self.out = torch.empty_like(self.q)
        self.lse = torch.empty(self.b, self.hq, self.t, dtype=torch.float32, device="cuda")
        self.dq, self.dk, self.dv = torch.empty_like(self.q), torch.empty_like(self.k), torch.empty_like(self.v)
        self.delta = torch.empty(self.hq, self.b * self.t, dtype=torch.float32, device="cuda")
        self.unit_flops = float(self.b) * self.hq * self.t * self.t * self.d

    def forward(self):
        self.fa.flash_attention_forward(self.q, self.k, self.v, out=self.out, lse=self.lse)

    def backward(self):
        self.fa.flash_attention_backward(self.q, self.k, self.v, self.out, self.lse, self.g, dq=self.dq, dk=self.dk,
                                         dv=self.dv, delta=self.delta)

    def step(self):
        self.forward()
        self.backward()

    def timed(self, fn, steps, warmup):
        torch = self.torch
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3  # ms per call

    def event_times(self, fn, steps):
        """Per-call durations (ms) from events on the launch stream (torch's current stream)."""
        torch = self.torch
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        for i in range(steps):
            starts[i].record()
            fn()
            stops[i].record()
        torch.cuda.synchronize()
        return sorted(a.elapsed_time(b) for a, b in zip(starts, stops))

    def kernel_times(self, steps):
        """Average duration of each kernel over `steps` timed steps (hipEvents on the launch stream)."""
        self.fa.set_kernel_timing(True)
        self.fa.collect_kernel_timings()
        for _ in range(steps):
            self.step()
        times = self.fa.collect_kernel_timings()
        self.fa.set_kernel_timing(False)
        return {k: total / max(n, 1) for k, (total, n) in times.items()}


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(name, heads_sample, full=False, loop_mode=True):
    """The CPU oracle (a restatement of the reference's OpenMP attention) timed in the two ways the reference runs it:
    one sequence at a time with the matrix products OpenMP-parallel inside ("single-call", Math/Matrix.cpp:139-146), and
    one thread per sequence of the batch with serial products ("train-loop", Network/LanguageModel.cpp:1109-1125).
    full: the whole configuration (every sequence and head); otherwise a bounded sample of `heads_sample` (batch, head)
    pairs of one sequence, with the time of the whole configuration extrapolated linearly (heads and sequences are
    independent on the CPU path) and labelled so."""
    import numpy as np
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib
    b, hq, hkv, t, d, dtype, sigma, _ = CONFIGS[name]
    group = hq // hkv
    heads_sample = hq if full else max(group, min(hq, heads_sample) // group * group)
    kv_sample = heads_sample // group
    packs_single = b if full else 1
    threads = oracle_lib.oracle().sentinel_oracle_max_threads()
    rng = np.random.default_rng(0x5E17)

    def draw(heads, kv_heads, packs):
        q = (sigma * rng.standard_normal((heads * d, packs * t))).astype(np.float32)
        k = (sigma * rng.standard_normal((kv_heads * d, packs * t))).astype(np.float32)
        v = rng.standard_normal((kv_heads * d, packs * t)).astype(np.float32)
        g = rng.standard_normal((heads * d, packs * t)).astype(np.float32)
        return q, k, v, g

    pair_flops = 7.0 * t * t * d  # one (batch, head) pair, causal count
    # single-call mode: the sequences one after the other, products parallel inside
    q, k, v, g = draw(heads_sample, kv_sample, packs_single)
    t0 = time.perf_counter()
    oracle_lib.oracle_attention(q, k, v, g, q_heads=heads_sample, kv_heads=kv_sample, head_dim=d, seq_len=t,
                                pack_count=packs_single, pack_parallel=False)
    dt = time.perf_counter() - t0
    pairs = packs_single * heads_sample
    report = {
        "value": pairs * pair_flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "cpu": cpu_model(),
        "sample": ("single-call mode: " + (f"the whole configuration, {pairs} (batch, head) pairs" if full else
                                           f"1 sequence x {heads_sample} of {b * hq} (batch, head) pairs of {name}") +
                   f", fp32, forward+backward, {dt:.2f} s, gemm/softmax OpenMP-parallel inside; same causal FLOP count "
                   "although the CPU path multiplies the full T x T"),
        "seconds": dt,
        "whole_config_seconds": dt * (b * hq) / pairs,
        "whole_config_seconds_is": "measured" if full else "extrapolated from the sample (pairs are independent)",
    }
    if loop_mode:
        # train-loop mode: the b sequences of the batch in parallel, serial products
        heads_loop = hq if full else group
        q, k, v, g = draw(heads_loop, heads_loop // group, b)
        t1 = time.perf_counter()
        oracle_lib.oracle_attention(q, k, v, g, q_heads=heads_loop, kv_heads=heads_loop // group, head_dim=d, seq_len=t,
                                    pack_count=b, pack_parallel=True)
        dt_loop = time.perf_counter() - t1
        report["train_loop_mode"] = {
            "value": b * heads_loop * pair_flops / dt_loop / 1e12, "unit": "TFLOP/s", "cores": min(threads, b),
            "seconds": dt_loop, "whole_config_seconds": dt_loop * hq / heads_loop,
            "whole_config_seconds_is": "measured" if full else "extrapolated from the sample (heads are independent)",
            "sample": f"{b} sequences in parallel (one thread each, serial products) x {heads_loop} of {hq} heads"}
    return report


def columns_path(torch, name, steps, separate, modes=None):
    """The same step through Sentinel's own tensor layout (fp32 [(head*d + dim), B*T]) with 16-bit arithmetic:
    what the drop-in costs on top of the kernels (layout / type conversion passes, optionally with the rotary
    embedding fused into them instead of four separate elementwise passes)."""
    import sentinel_amd
    from sentinel_amd import HipFlashAttention, HipOps
    b, hq, hkv, t, d, dtype, sigma, _ = CONFIGS[name]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5E17 + 40)
    cols = b * t
    q = sigma * torch.randn(hq * d, cols, device="cuda", generator=gen)
    k = sigma * torch.randn(hkv * d, cols, device="cuda", generator=gen)
    v = torch.randn(hkv * d, cols, device="cuda", generator=gen)
    g = torch.randn(hq * d, cols, device="cuda", generator=gen)
    pos = torch.arange(t, device="cuda", dtype=torch.float32)[:, None]
    inv = torch.pow(torch.tensor(10000.0, device="cuda"), -2.0 * torch.arange(d // 2, device="cuda") / d)[None, :]
    cos, sin = torch.cos(pos * inv).contiguous(), torch.sin(pos * inv).contiguous()
    scale = 1.0 / d ** 0.5
    args = (hq, d, scale, True, 0, t, b)
    state = {"out": None, "lse": None, "dq": None, "dk": None, "dv": None, "delta": None, "ws": None}
    lib = sentinel_amd.load_library()
    need = lib.sentinel_hip_flash_workspace_bytes(0, {"bf16": 1, "fp16": 2}[dtype], 0, hq, hkv, d, t, b, 1)
    state["ws"] = torch.empty(need, dtype=torch.uint8, device="cuda")

    def step(mode):
        kw = dict(kv_head_count=hkv, compute=dtype, workspace=state["ws"])
        fkw, bkw = {}, {}
        if mode in ("fused", "fused_kept"):
            kw["rope"] = (cos, sin)
        if mode in ("plain_kept", "fused_kept"):  # the forward leaves its 16-bit operands in the workspace for the backward
            fkw, bkw = {"keep_for_backward": True}, {"reuse_forward_workspace": True}
        if mode == "separate":  # the reference's sequence: rotate Q, K in place, attend, rotate dQ, dK back
            HipOps.rotary_rotate_in_place(q, hq, d, d // 2, cos, sin, 0, t)
            HipOps.rotary_rotate_in_place(k, hkv, d, d // 2, cos, sin, 0, t)
        state["out"], state["lse"] = HipFlashAttention.forward_multi_head(q, k, v, state["out"], state["lse"], *args, **kw,
                                                                          **fkw)
        state["dq"], state["dk"], state["dv"], state["delta"] = HipFlashAttention.backward_multi_head(
            q, k, v, state["out"], state["lse"], g, state["dq"], state["dk"], state["dv"], state["delta"], *args, **kw, **bkw)
        if mode == "separate":
            HipOps.rotary_rotate_inverse_in_place(state["dq"], hq, d, d // 2, cos, sin, 0, t)
            HipOps.rotary_rotate_inverse_in_place(state["dk"], hkv, d, d // 2, cos, sin, 0, t)
            HipOps.rotary_rotate_inverse_in_place(q, hq, d, d // 2, cos, sin, 0, t)  # restore the inputs
            HipOps.rotary_rotate_inverse_in_place(k, hkv, d, d // 2, cos, sin, 0, t)

    report = {}
    if modes is None:
        modes = ("plain", "plain_kept", "fused", "fused_kept") + (("separate",) if separate else ())
    for mode in modes:
        for _ in range(2):
            step(mode)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step(mode)
        torch.cuda.synchronize()
        report[mode + "_ms_per_step"] = (time.perf_counter() - t0) / steps * 1e3
    sentinel_amd.set_kernel_timing(True)
    sentinel_amd.collect_kernel_timings()
    for _ in range(steps):
        step("fused_kept")
    times = sentinel_amd.collect_kernel_timings()
    sentinel_amd.set_kernel_timing(False)
    report["kernels_ms"] = {kname: tot / max(n, 1) for kname, (tot, n) in times.items()}
    for kname in ("columns_to_bhtd", "bhtd_to_columns"):  # conversion passes: 4 + 2 bytes per element
        if kname in times:
            report[kname + "_avg_ms"] = times[kname][0] / max(times[kname][1], 1)
    elems = float(hq * d) * cols
    flops = 7.0 * float(b) * hq * t * t * d
    for mode in modes:
        report[mode + "_tflops"] = flops / (report[mode + "_ms_per_step"] * 1e-3) / 1e12
    report["note"] = ("fp32 [(head*d + dim), B*T] tensors, 16-bit arithmetic; plain = unrotated call; fused = rotary embedding "
                      "inside the conversion passes; *_kept = the forward call leaves its 16-bit operands in the workspace "
                      "and the backward call converts d_out only (kernels_ms is this mode); separate = rotate Q, K in place "
                      "+ plain step + rotate dQ, dK back (+ restoring Q, K: 4 extra passes that a real caller does not need)")
    report["elements_per_q_tensor"] = elems
    return report


def decode_path(torch, steps):
    """The generation step's attention (one query column against the K/V cache, Sentinel's cache layout) against
    the HBM roofline: algorithmic bytes = the used prefix of the K and V caches, 2 * kv_heads * d * length * 4,
    read once, over the HIP-event time of the two launches (split scores / partial outputs, then the merge)."""
    import sentinel_amd
    lib = sentinel_amd.load_library()
    report = {}
    for label, (hq, hkv, d, length) in {
        "gqa_32q_8kv_d128_L32768": (32, 8, 128, 32768),
        "mha_32_d128_L4096": (32, 32, 128, 4096),
        "gqa_32q_8kv_d128_L4096": (32, 8, 128, 4096),
        "mha_16_d64_L16384": (16, 16, 64, 16384),
        "mha_12_d64_L1024": (12, 12, 64, 1024),
    }.items():
        gen = torch.Generator(device="cuda")
        gen.manual_seed(0x5E17 + length)
        q = torch.randn(hq * d, 1, device="cuda", generator=gen)
        k = torch.randn(hkv * d, length, device="cuda", generator=gen)
        v = torch.randn(hkv * d, length, device="cuda", generator=gen)
        out = torch.empty_like(q)
        ws = torch.empty(lib.sentinel_hip_decode_workspace_bytes(hq, d, length) + 16, dtype=torch.uint8, device="cuda")
        call = lambda: sentinel_amd.decode_attention(q, k, v, length, hq, d, kv_head_count=hkv, out=out, workspace=ws)
        for _ in range(5):
            call()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            call()
        torch.cuda.synchronize()
        wall_us = (time.perf_counter() - t0) / steps * 1e6
        sentinel_amd.set_kernel_timing(True)
        sentinel_amd.collect_kernel_timings()
        for _ in range(steps):
            call()
        times = sentinel_amd.collect_kernel_timings()
        sentinel_amd.set_kernel_timing(False)
        partial_us = times["decode_partial"][0] / times["decode_partial"][1] * 1e3
        merge_us = times["decode_merge"][0] / times["decode_merge"][1] * 1e3
        cache_bytes = 2.0 * hkv * d * length * 4
        achieved = cache_bytes / ((partial_us + merge_us) * 1e-6) / 1e9
        report[label] = {"q_heads": hq, "kv_heads": hkv, "head_dim": d, "length": length, "cache_bytes": cache_bytes,
                         "partial_us": partial_us, "merge_us": merge_us, "call_us_back_to_back": wall_us,
                         "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                      "frac": achieved / HBM_PEAK_GBS, "traffic": None}}
    return report


def sparse_path(torch, name, steps):
    """The step under the attention layer's sliding-window + global-token mask at the same shape: time and the
    matrix-core rate on the visible (query, key) pairs only, 14 * d FLOPs per pair (7 products of 2 * d)."""
    import sentinel_amd
    b, hq, hkv, t, d, dtype, _, _ = CONFIGS[name]
    q, k, v, g = make_inputs(torch, name)
    out = torch.empty_like(q)
    lse = torch.empty(b, hq, t, dtype=torch.float32, device="cuda")
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    delta = torch.empty(hq, b * t, dtype=torch.float32, device="cuda")
    report = {}
    for window, global_tokens in ((t // 8, 0), (t // 8, 64), (t // 32, 0), (t // 2, 0)):
        kw = dict(window_size=window, global_token_count=global_tokens)

        def step():
            sentinel_amd.flash_attention_forward(q, k, v, out=out, lse=lse, **kw)
            sentinel_amd.flash_attention_backward(q, k, v, out, lse, g, dq=dq, dk=dk, dv=dv, delta=delta, **kw)

        for _ in range(3):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / steps * 1e3
        sentinel_amd.set_kernel_timing(True)
        sentinel_amd.collect_kernel_timings()
        for _ in range(steps):
            step()
        times = sentinel_amd.collect_kernel_timings()
        sentinel_amd.set_kernel_timing(False)
        pairs = sum(min(qi + 1, window) + min(global_tokens, max(qi + 1 - window, 0)) for qi in range(t))
        flops = 14.0 * d * pairs * b * hq
        report[f"W{window}_G{global_tokens}"] = {
            "ms_per_step": ms, "visible_pairs_fraction_of_causal": pairs / (t * (t + 1) / 2.0),
            "tflops_on_visible_pairs": flops / (ms * 1e-3) / 1e12,
            "kernels_ms": {kname: tot / max(n, 1) for kname, (tot, n) in times.items()}}
    return report


def library_gemm(torch, dtype, n=8192, calls=30):
    """The vendor library's plain n^3 GEMM (torch.matmul -> hipBLASLt) in the workload's 16-bit type, timed like the
    kernels: the matrix throughput this box sustains on a full-chip GEMM under its clock and power management, to read
    the attention kernels' fraction of the nominal peak against."""
    tdt = {"bf16": torch.bfloat16, "fp16": torch.float16}[dtype]
    a = torch.randn(n, n, device="cuda").to(tdt)
    b = torch.randn(n, n, device="cuda").to(tdt)
    c = torch.empty(n, n, device="cuda", dtype=tdt)
    for _ in range(5):
        torch.matmul(a, b, out=c)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(calls):
        torch.matmul(a, b, out=c)
    stop.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(stop) / calls
    tf = 2.0 * n ** 3 / (ms * 1e-3) / 1e12
    return {"shape": [n, n, n], "dtype": dtype, "ms": ms, "tflops": tf, "pct_of_mfma_peak": 100.0 * tf / PEAK_TFLOPS[dtype]}


def profiler_attached():
    """True under rocprofv3 (its preloaded tool library has initialised the GPU before this program started, and a
    process that has done so must not start another program)."""
    env = os.environ
    return "rocprof" in env.get("LD_PRELOAD", "").lower() or any(k.startswith(("ROCPROF", "ROCP_")) for k in env)


def layer_path(columns, steps):
    """The attention layer behind the reference's class interface (include/sentinel_hip/HipCausalSelfAttention.hpp:
    projections, rotation, attention core, output projection and their backward) with flash attention on and off, on
    the reference's flash-parity shapes, and with the projection products in mixed precision as well
    (flash_mixed_projections): the "attention fwd/bwd ms" of its train profile.  Timed by the C++ program
    tests/cpp/bench_layer (the layer is C++), started as a child process before this process touches the GPU."""
    import subprocess
    exe = os.path.join(ROOT, "tests", "cpp", "bench_layer")
    if not os.path.exists(exe):
        return {"skipped": "tests/cpp/bench_layer is not built (python -c 'import __graft_entry__ as g; g.build()')"}
    try:
        proc = subprocess.run([exe, str(columns), str(steps), "3"], capture_output=True, text=True, timeout=240)
    except (OSError, subprocess.SubprocessError) as exc:
        return {"skipped": f"bench_layer did not run: {exc}"}
    if proc.returncode != 0:
        return {"skipped": f"bench_layer exit code {proc.returncode}: {proc.stderr.strip()[-300:]}"}
    return json.loads(proc.stdout.strip().splitlines()[-1])


def rocminfo_gpu_clock_ghz():
    """Max Clock Freq. of the first gfx agent as printed by rocminfo (GHz), 0.0 if it cannot be read."""
    import re
    import subprocess
    try:
        text = subprocess.run(["/opt/rocm/bin/rocminfo"], capture_output=True, text=True, timeout=30).stdout
    except (OSError, subprocess.SubprocessError):
        return 0.0
    for block in text.split("*******")[1:]:
        if re.search(r"Name:\s+gfx", block):
            m = re.search(r"Max Clock Freq\. \(MHz\):\s+(\d+)", block)
            if m:
                return int(m.group(1)) / 1e3
    return 0.0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="nstar", choices=sorted(CONFIGS))
    ap.add_argument("--cpu-heads", type=int, default=8, help="(batch, head) pairs in the CPU baseline sample; 0 = skip")
    ap.add_argument("--no-configs", action="store_true", help="skip the brief timing of the other configurations")
    ap.add_argument("--no-columns-path", action="store_true",
                    help="skip timing the step through Sentinel's fp32 column layout (conversion passes, fused rotary "
                         "embedding), reported under \"columns_path\"")
    ap.add_argument("--columns-separate-rope", action="store_true",
                    help="columns_path also times the reference's sequence of separate in-place rotary passes")
    ap.add_argument("--no-layer-path", action="store_true",
                    help="skip timing the C++ attention layer with flash attention on and off (\"layer_path\"; a child "
                         "process, started first; skipped by itself under a profiler)")
    ap.add_argument("--layer-columns", type=int, default=4096, help="tokens per step of the layer timing")
    ap.add_argument("--sparse-path", action="store_true",
                    help="also time the step under sliding-window + global-token masks and report it under \"sparse_path\"")
    ap.add_argument("--decode-path", action="store_true",
                    help="also time single-query attention against a K/V cache (generation) and report it under \"decode_path\"")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB -> 1 GiB elementwise copy kernel three times, so that a counter run "
                         "(FETCH_SIZE / WRITE_SIZE) of this command holds a kernel of known traffic to scale by")
    ap.add_argument("--no-gemm-calibration", action="store_true",
                    help="skip timing the vendor library's plain 8192^3 16-bit GEMM (\"device.library_gemm\": what the "
                         "matrix pipes of this very box sustain under its power limit; skipped by itself under a profiler)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU only; attention shards over (batch, kv-head group) with no "
              "exchange, so a multi-GPU figure would be N independent copies of this one", file=sys.stderr)
        sys.exit(2)

    # child processes first: nothing may be started once this process has initialised the GPU
    layer = None
    if not args.no_layer_path:
        layer = ({"skipped": "a profiler is attached"} if profiler_attached()
                 else layer_path(args.layer_columns, max(args.steps // 2, 5)))
    fallback_clock_ghz = rocminfo_gpu_clock_ghz() if not profiler_attached() else 0.0

    import torch
    import sentinel_amd
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    sentinel_amd.load_library()

    props = torch.cuda.get_device_properties(0)
    cus = int(props.multi_processor_count)
    clock_ghz = float(getattr(props, "clock_rate", 0)) / 1e6  # kHz -> GHz
    if clock_ghz <= 0.0:  # not filled in by this torch build: what rocminfo printed for the GPU agent's maximum clock
        clock_ghz = fallback_clock_ghz
    device = {"name": props.name, "compute_units": cus, "max_clock_ghz": clock_ghz,
              # dense bf16 / fp16 MFMA: 4096 FLOP per clock per CU; the fraction below uses the published figure
              "mfma_peak_from_device_tflops": cus * 4096 * clock_ghz / 1e3}

    w = Workload(torch, args.config)
    ms_step = w.timed(w.step, args.steps, args.warmup)
    ev_step = w.event_times(w.step, args.steps)
    ev_fwd = w.event_times(w.forward, args.steps)
    ev_bwd = w.event_times(w.backward, args.steps)
    ms_fwd = ev_fwd[len(ev_fwd) // 2]
    ms_bwd = ev_bwd[len(ev_bwd) // 2]
    kernels = w.kernel_times(min(args.steps, 20))
    if args.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")  # 1 GiB read, 1 GiB written per launch
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
    if not args.no_gemm_calibration and not profiler_attached() and w.dtype != "fp32":
        device["library_gemm"] = library_gemm(torch, w.dtype)
    total_flops = 7.0 * w.unit_flops
    value = total_flops / (ms_step * 1e-3) / 1e12
    peak = PEAK_TFLOPS[w.dtype]

    counted = {k: v for k, v in kernels.items() if k in KERNEL_UNITS}
    dominant = max(counted, key=counted.get)
    achieved = KERNEL_UNITS[dominant] * w.unit_flops / (counted[dominant] * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": dominant, "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                "frac": achieved / peak, "traffic": measured_traffic_bytes(args.config, dominant),
                "kernel_ms": counted[dominant],
                "algorithmic_flops_per_launch": KERNEL_UNITS[dominant] * w.unit_flops}

    line = {
        "metric": "causal flash-attn fwd+bwd TFLOP/s",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w.dtype,
        "data": "synthetic",
        "config": {"workload": w.desc, "batch": w.b, "q_heads": w.hq, "kv_heads": w.hkv, "seq_len": w.t, "head_dim": w.d,
                   "causal": True, "layout": "[B,H,T,d]"},
        "pct_of_mfma_peak": 100.0 * value / peak,
        "fwd_ms": ms_fwd,
        "bwd_ms": ms_bwd,
        "fwd_tflops": 2.0 * w.unit_flops / (ms_fwd * 1e-3) / 1e12,
        "bwd_tflops": 5.0 * w.unit_flops / (ms_bwd * 1e-3) / 1e12,
        "step_ms_median_min": [ev_step[len(ev_step) // 2], ev_step[0]],
        "fwd_ms_median_min": [ms_fwd, ev_fwd[0]],
        "bwd_ms_median_min": [ms_bwd, ev_bwd[0]],
        "timing": "value: wall clock over the timed steps; *_median_min: per-call events on the launch stream; "
                  "buffers allocated once, L2 not flushed",
        "device": device,
        "kernels_ms": kernels,
        "roofline": roofline,
    }

    if not args.no_configs:
        others = {}
        for name in ("c1", "c2", "c3", "c4", "c5"):
            if name == args.config:
                continue
            o = Workload(torch, name)
            steps = 10 if name != "c1" else 50
            f_ms = o.timed(o.forward, steps, 2)
            b_ms = o.timed(o.backward, steps, 2)
            tf = 7.0 * o.unit_flops / ((f_ms + b_ms) * 1e-3) / 1e12
            others[name] = {"workload": o.desc, "dtype": o.dtype, "fwd_ms": f_ms, "bwd_ms": b_ms, "tflops": tf,
                            "pct_of_mfma_peak": 100.0 * tf / PEAK_TFLOPS[o.dtype]}
            del o
            torch.cuda.empty_cache()
        if "c2" in others and not args.no_columns_path:
            # the drop-in path at the shape Sentinel itself trains with (fp32 column matrices, rotation fused, operands kept)
            cp = columns_path(torch, "c2", 20, separate=False, modes=("fused_kept",))
            cp["native_ms_per_step"] = others["c2"]["fwd_ms"] + others["c2"]["bwd_ms"]
            cp["over_native"] = cp["fused_kept_ms_per_step"] / cp["native_ms_per_step"]
            others["c2"]["columns_path"] = cp
        line["configs"] = others

    if not args.no_columns_path and w.dtype != "fp32":
        del w
        torch.cuda.empty_cache()
        line["columns_path"] = columns_path(torch, args.config, max(args.steps // 5, 3), separate=args.columns_separate_rope)

    if args.sparse_path:
        line["sparse_path"] = sparse_path(torch, args.config, max(args.steps // 2, 5))

    if args.decode_path:
        line["decode_path"] = decode_path(torch, max(args.steps, 20))

    if layer is not None:
        line["layer_path"] = layer

    if args.cpu_heads > 0:
        line["cpu_baseline"] = cpu_baseline(args.config, args.cpu_heads)
        # every other configuration next to its own CPU time: C1 and C2 whole, both modes; the long ones one
        # (batch, head) pair of one sequence in single-call mode, extrapolated
        for name, entry in line.get("configs", {}).items():
            entry["cpu_baseline"] = (cpu_baseline(name, 0, full=True) if name in ("c1", "c2")
                                     else cpu_baseline(name, 1, loop_mode=False))
            entry["speedup_over_cpu_single_call"] = (entry["cpu_baseline"]["whole_config_seconds"] /
                                                     ((entry["fwd_ms"] + entry["bwd_ms"]) * 1e-3))
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
