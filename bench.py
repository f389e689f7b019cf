#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-details] [--no-cpu]

Headline (the ONE JSON line printed last): the SmoothQuant W8A8 sweep at Qwen2-7B shapes -
projections qkv / o / gate_up / down at M in {1, 16, 128, 2048, 8192}, each linear = per-token
dynamic int8 quantizer kernel + int8 MFMA GEMM with the per-token x per-channel dequant epilogue.
A "step" is one pass over those 20 linears with every input already resident in HBM; `value` is
sum(2*M*N*K) / step time in TOPS.  The same line carries
  roofline     - the dominant kernel (int8 MFMA GEMM at the prefill shapes M >= 2048), timed per
                 launch with HIP events on the launch stream, against the dense int8 MFMA peak;
  cpu_baseline - the reference's dequantize-then-matmul math (the oracle) on the host cores for a
                 bounded sample of the same workload, which also serves as the parity check;
  details      - per-shape figures for the W8A8 sweep, the FP8 sweep, AWQ W4A16 decode (GB/s
                 against the HBM peak) and the decoder-layer stack.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)



def _profile_traffic(summary):
    """HBM-side bytes per launch of a kernel, averaged over the launches of its roofline leg: FETCH_SIZE and WRITE_SIZE
    of two `rocprofv3 --pmc` runs of this file's profiler mode, each scaled by what the same counter reads for the
    256 MiB calibration copy.  Counters cannot be read from inside this process, so the figure is taken from the
    `TRAFFIC_BYTES_PER_LAUNCH=` line of the tracked summary that was made from those runs; None when there is none."""
    try:
        with open(os.path.join(ROOT, "profiles", summary)) as f:
            for line in f:
                if line.startswith("TRAFFIC_BYTES_PER_LAUNCH="):
                    return int(line.split("=", 1)[1])
    except OSError:
        pass
    return None


ROOFLINE_TRAFFIC_BYTES = _profile_traffic("gemm_w8a8_int8_mfma_prefill_qwen2_7b.md")   # bench.py --roofline-only
FP8_TRAFFIC_BYTES = _profile_traffic("gemm_fp8_mfma_prefill_qwen2_7b.md")               # bench.py --fp8-only
W4A16_TRAFFIC_BYTES = _profile_traffic("awq_gemv_w4a16_decode_qwen2_7b.md")             # bench.py --awq-only, M <= 16
CPU_BASELINE_REPS = 12        # bounded CPU sample: about 10-15 s of host work
PEAK_INT8_TOPS = 5033.0   # dense int8 MFMA peak of MI355X, TOP/s (256 CU x 2.4 GHz x 8192 op/clk)
PEAK_FP8_TFLOPS = 5033.0  # dense fp8 MFMA peak
PEAK_HBM_GBS = 8000.0     # HBM3E peak, GB/s


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-details", action="store_true", help="skip the per-shape FP8 / AWQ / layer tables")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--awq-only", action="store_true",
                    help="profiler mode: only the W4A16 launches of configs[3] (4 projections x M in {1,4,16,64}), "
                         "weights rotated beyond the Infinity Cache, preceded by one 256 MiB calibration copy")
    ap.add_argument("--awq-prefill-only", action="store_true",
                    help="profiler mode: only the W4A16 tile kernel (4 projections x M in {128,256,512,2048}), "
                         "preceded by one 256 MiB calibration copy")
    ap.add_argument("--quant-only", action="store_true",
                    help="profiler mode: only the row kernels (int8 / fp8 per-token quantizers, RMSNorm, RMSNorm fused "
                         "with the int8 quantizer) at M in {2048, 8192} x K in {3584, 18944}, after one 256 MiB copy")
    ap.add_argument("--fp8-only", action="store_true",
                    help="profiler mode: only the FP8 GEMM launches (4 projections x M in {512, 4096}), preceded by "
                         "one 256 MiB calibration copy")
    ap.add_argument("--micro", action="store_true",
                    help="hardware microbenchmarks instead of the workload: register-only MFMA rate (random / zero "
                         "operands), LDS bandwidth per CU, and HBM streaming rate of a packed W4 matrix by access pattern")
    ap.add_argument("--roofline-only", action="store_true",
                    help="run only the dominant kernel's launches (for rocprofv3 summaries)")
    return ap.parse_args()


class W8A8Linear:
    """One W8A8 linear with preallocated buffers; launch() = quantizer + GEMM through the C ABI."""

    def __init__(self, name, M, K, N, qweight, w_scale, seed, dev, x=None, norm_weight=None, eps=1e-6):
        from llmqrt_amd import _abi, workloads as W
        self.name, self.M, self.K, self.N = name, M, K, N
        self.x = (W.activations(M, K, seed) if x is None else x).to(dev)
        self.norm_weight, self.eps = norm_weight, eps   # set: RMSNorm fused into the quantizer launch
        self.qweight, self.w_scale = qweight, w_scale
        self.qx = torch.empty((M, K), dtype=torch.int8, device=dev)
        self.a_scale = torch.empty((M,), dtype=torch.float32, device=dev)
        self.out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        L = _abi.lib()
        ws_bytes = L.llmq_gemm_workspace_bytes(M, N, K)
        self.ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        self.ws_bytes = ws_bytes
        self.L, self.abi = L, _abi
        self.ops = 2 * M * N * K

    def quant(self, stream):
        if self.norm_weight is not None:
            return self.L.llmq_rmsnorm_quant_i8_per_token(self.x.data_ptr(), self.abi.BF16, self.M, self.K, self.K,
                                                          self.norm_weight.data_ptr(), self.eps, None,
                                                          self.qx.data_ptr(), self.a_scale.data_ptr(), self.abi.F32,
                                                          None, stream)
        return self.L.llmq_quant_i8_per_token(self.x.data_ptr(), self.abi.BF16, self.M, self.K, self.K,
                                              self.qx.data_ptr(), self.a_scale.data_ptr(), self.abi.F32, stream)

    def gemm(self, stream, acc_dump=None):
        return self.L.llmq_gemm_w8a8(self.qx.data_ptr(), self.K, self.qweight.data_ptr(), self.K,
                                     self.a_scale.data_ptr(), self.w_scale.data_ptr(), 1.0, None, None, 0, 0.0,
                                     self.out.data_ptr(), self.abi.BF16, self.N, self.M, self.N, self.K,
                                     acc_dump, self.ws.data_ptr(), self.ws.numel(), stream)

    def launch(self, stream):
        rc = self.quant(stream)
        rc |= self.gemm(stream)
        return rc


def event_time_us(fn, stream_obj, reps):
    """Average duration of fn() in microseconds from HIP events recorded on the launch stream."""
    fn()
    stream_obj.synchronize()
    times = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream_obj)
        fn()
        e1.record(stream_obj)
        e1.synchronize()
        times.append(e0.elapsed_time(e1) * 1e3)
    return statistics.mean(times), min(times)


def batch_time_us(fns, stream_obj, reps, rounds=5):
    """Median over `rounds` batches of the per-launch time of back-to-back launches cycling through `fns`,
    after 10 warm-up launches; short kernels (< 100 us) are timed over at least 100 launches per batch."""
    for i in range(10):
        fns[i % len(fns)]()
    stream_obj.synchronize()
    per = []
    for r in range(rounds + 1):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream_obj)
        for i in range(reps):
            fns[i % len(fns)]()
        e1.record(stream_obj)
        e1.synchronize()
        t = e0.elapsed_time(e1) * 1e3 / reps
        if r == 0:
            if t < 100.0:
                reps = max(reps, 100)
            continue  # the first batch only sizes the later ones
        per.append(t)
    return statistics.median(per)


def sequence_time_us(launches, stream_obj, passes):
    """The launches of a roofline leg back to back in a fixed order, as the profiler modes run them (`passes` times
    after one untimed pass), every launch bracketed by HIP events on the launch stream and no host synchronisation
    inside a pass.  launches: [(name, fn(pass_index))].  -> {name: mean microseconds}."""
    for _, fn in launches:
        fn(0)
    torch.cuda.synchronize()
    times = {name: [] for name, _ in launches}
    for it in range(passes):
        evs = []
        for name, fn in launches:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream_obj)
            fn(it + 1)
            e1.record(stream_obj)
            evs.append((name, e0, e1))
        torch.cuda.synchronize()
        for name, e0, e1 in evs:
            times[name].append(e0.elapsed_time(e1) * 1e3)
    return {name: statistics.mean(v) for name, v in times.items()}


def build_w8a8_sweep(dev):
    from llmqrt_amd import workloads as W
    linears = []
    for pi, (pname, (K, N)) in enumerate(W.QWEN2_7B_PROJ.items()):
        qw, ws = W.int8_weights(N, K, W.seed_for(1, 100 + pi))
        qw, ws = qw.to(dev), ws.to(dev)
        for mi, M in enumerate(W.W8A8_M):
            linears.append(W8A8Linear(f"{pname}_M{M}", M, K, N, qw, ws, W.seed_for(1, 10 * pi + mi), dev))
    # big launches first so that the queue stays full while the host enqueues the small ones
    linears.sort(key=lambda l: -l.ops)
    return linears


def cpu_baseline_and_parity(linears, dev):
    """The oracle (dequantize-then-matmul, reference linear_sq.py:117-125) timed on the host cores
    for the four projections at M = 2048, and used as the checker of the GPU results."""
    from oracle import ref_math as R
    sample = [l for l in linears if l.M == 2048]
    stream = torch.cuda.current_stream().cuda_stream
    total_ops, total_s, worst_rel, acc_exact = 0, 0.0, 0.0, True
    for l in sample:
        dump = torch.empty((l.M, l.N), dtype=torch.int32, device=dev)
        l.quant(stream)
        l.gemm(stream, dump.data_ptr())
        torch.cuda.synchronize()
        x_cpu, qw_cpu, ws_cpu = l.x.cpu(), l.qweight.cpu(), l.w_scale.cpu()
        for _ in range(CPU_BASELINE_REPS):  # ~1 s per pass over the four projections on 16 threads
            t0 = time.perf_counter()
            qx, sx = R.quantize_activation_per_token_absmax(x_cpu)
            y = R.w8a8_linear_naive(qx, sx, qw_cpu, ws_cpu, None, torch.bfloat16)
            total_s += time.perf_counter() - t0
            total_ops += l.ops
        # checker (not timed): quantizer bit-exact, 64 sampled accumulator rows bit-exact, output tolerance
        acc_exact &= torch.equal(l.qx.cpu(), qx) and torch.equal(l.a_scale.cpu(), sx.float().view(-1))
        rows = torch.arange(0, l.M, l.M // 64)
        acc_exact &= torch.equal(dump.cpu()[rows], R.int8_gemm_exact(qx[rows], qw_cpu))
        rel = ((l.out.float().cpu() - y.float()).abs().max() / y.float().abs().max()).item()
        worst_rel = max(worst_rel, rel)
    return {
        "value": round(total_ops / total_s / 1e12, 4), "unit": "TOPS", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "per-token int8 quantizer + dequantize-then-matmul (torch fp32, oracle/ref_math.py) of the 4 "
                  "Qwen2-7B projections at M=2048, %d repetitions, %d host threads of %d cores" %
                  (CPU_BASELINE_REPS, torch.get_num_threads(), os.cpu_count()),
        "seconds": round(total_s, 2),
    }, {"int32_acc_and_quantizer_bit_exact": bool(acc_exact), "max_rel_err_vs_oracle": worst_rel, "tolerance": 1e-2}


def details_fp8(dev):
    from llmqrt_amd import _abi, workloads as W
    L = _abi.lib()
    stream_obj = torch.cuda.current_stream()
    stream = stream_obj.cuda_stream
    rows = []
    for pi, (pname, (K, N)) in enumerate(W.QWEN2_7B_PROJ.items()):
        wq, ws = W.fp8_weights(N, K, W.seed_for(2, 100 + pi))
        wq, ws = wq.to(dev), ws.to(dev)
        for mi, M in enumerate(W.FP8_M):
            x = W.activations(M, K, W.seed_for(2, 10 * pi + mi)).to(dev)
            xq = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=dev)
            xs = torch.empty((M,), dtype=torch.float32, device=dev)
            out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
            wsb = L.llmq_gemm_workspace_bytes(M, N, K)
            wsp = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)

            def quant():
                L.llmq_quant_fp8_per_token(x.data_ptr(), _abi.BF16, M, K, K, xq.data_ptr(), xs.data_ptr(), stream)

            def gemm():
                L.llmq_gemm_fp8(xq.data_ptr(), _abi.E4M3, K, wq.data_ptr(), K, xs.data_ptr(), ws.data_ptr(), 1.0, None,
                                None, 0, 0.0, out.data_ptr(), _abi.BF16, N, M, N, K, None, wsp.data_ptr(), wsp.numel(),
                                stream)
            quant()
            t_gemm = batch_time_us([gemm], stream_obj, 20)
            t_quant = batch_time_us([quant], stream_obj, 20)
            tflops = 2 * M * N * K / t_gemm / 1e6
            rows.append({"proj": pname, "M": M, "gemm_us": round(t_gemm, 2), "quant_us": round(t_quant, 2),
                         "gemm_TFLOPS": round(tflops, 1), "pct_fp8_mfma_peak": round(100 * tflops / PEAK_FP8_TFLOPS, 2),
                         "gemm_GBs": round(W.w8a8_gemm_bytes(M, N, K) / t_gemm / 1e3, 1)})
    return rows


FP8_PREFILL_M = (512, 4096)


def fp8_launch_set(dev):
    """The FP8 GEMM launches at the prefill sizes of configs[2] in a fixed order, activations quantized once.
    -> [(name, M, N, K, fn(pass_index))]"""
    from llmqrt_amd import _abi, workloads as W
    L = _abi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    launches = []
    for pi, (pname, (K, N)) in enumerate(W.QWEN2_7B_PROJ.items()):
        wq, ws = (t.to(dev) for t in W.fp8_weights(N, K, W.seed_for(2, 100 + pi)))
        for M in FP8_PREFILL_M:
            mi = W.FP8_M.index(M)
            x = W.activations(M, K, W.seed_for(2, 10 * pi + mi)).to(dev)
            xq = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=dev)
            xs = torch.empty((M,), dtype=torch.float32, device=dev)
            out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
            wsp = torch.empty(max(L.llmq_gemm_workspace_bytes(M, N, K), 16), dtype=torch.uint8, device=dev)
            assert L.llmq_quant_fp8_per_token(x.data_ptr(), _abi.BF16, M, K, K, xq.data_ptr(), xs.data_ptr(), stream) == 0

            def fn(it, a=(xq, xs, wq, ws, out, wsp, M, N, K)):
                xq_, xs_, wq_, ws_, out_, wsp_, M_, N_, K_ = a
                rc = L.llmq_gemm_fp8(xq_.data_ptr(), _abi.E4M3, K_, wq_.data_ptr(), K_, xs_.data_ptr(), ws_.data_ptr(), 1.0,
                                     None, None, 0, 0.0, out_.data_ptr(), _abi.BF16, N_, M_, N_, K_, None, wsp_.data_ptr(),
                                     wsp_.numel(), stream)
                assert rc == 0
            launches.append((f"{pname}_M{M}", M, N, K, fn))
    torch.cuda.synchronize()
    return launches


def fp8_only(dev, steps, warmup):
    """For profiler runs: the launches of fp8_launch_set after one plain copy of known size that calibrates the HBM
    byte counters."""
    cal_src = torch.zeros(64 << 20, dtype=torch.int32, device=dev)
    cal_dst = torch.empty_like(cal_src)
    launches = fp8_launch_set(dev)
    cal_dst.copy_(cal_src)
    for it in range(warmup + steps):
        for _, _, _, _, fn in launches:
            fn(it)
        if it + 1 == warmup:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    print(json.dumps({"fp8_only": True, "order": [l[0] for l in launches], "steps": steps, "warmup": warmup,
                      "calibration_copy_bytes_each_way": cal_src.numel() * 4}))


def roofline_fp8(dev, passes):
    """FP8 GEMM at the prefill sizes (M >= 512) of configs[2]: sum(2MNK) over the sum of the launch durations, timed in
    the launch sequence of `--fp8-only` (the one the tracked profiler summary traces)."""
    from llmqrt_amd import workloads as W
    launches = fp8_launch_set(dev)
    us = sequence_time_us([(l[0], l[4]) for l in launches], torch.cuda.current_stream(), passes)
    ops = sum(2 * M * N * K for _, M, N, K, _ in launches)
    alg = sum(W.w8a8_gemm_bytes(M, N, K) for _, M, N, K, _ in launches)
    tot = sum(us.values())
    ach = ops / tot / 1e6
    return {"bound": "mfma", "achieved": round(ach, 1), "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
            "frac": round(ach / PEAK_FP8_TFLOPS, 4), "traffic": FP8_TRAFFIC_BYTES,
            "algorithmic_bytes": alg // len(launches),
            "kernel": "gemm_tile_kernel<fp8 e4m3> at M in {512, 4096} x {qkv, o, gate_up, down}",
            "avg_launch_us": round(tot / len(launches), 2),
            "launches": [{"shape": n, "us": round(us[n], 2), "TFLOPS": round(2 * M * N * K / us[n] / 1e6, 1)}
                         for n, M, N, K, _ in launches]}


def awq_launch_set(dev, token_counts):
    """The W4A16 launches of configs[3] for the given token counts in a fixed order; pass i reads copy i of the weights,
    which rotate through more than 256 MB per projection so that the Infinity Cache cannot hold them.
    -> [(name, M, N, K, fn(pass_index))]"""
    from llmqrt_amd import _abi, workloads as W
    L = _abi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    launches = []
    for pi, (pname, (K, N)) in enumerate(W.QWEN2_7B_PROJ.items()):
        qw, qz, sc = W.awq_weights(N, K, W.seed_for(3, 100 + pi))
        wbytes = qw.numel() * 4 + qz.numel() * 4 + sc.numel() * 2
        ncopies = max(2, -(-320 * 1024 * 1024 // wbytes))
        copies = [(qw.to(dev).clone(), qz.to(dev).clone(), sc.to(dev).clone()) for _ in range(ncopies)]
        for M in token_counts:
            mi = W.AWQ_M.index(M)
            x = W.activations(M, K, W.seed_for(3, 10 * pi + mi), dtype=torch.float16, outliers=False).to(dev)
            out = torch.empty((M, N), dtype=torch.float16, device=dev)
            # the arrival counters at the start of the workspace are cleared once, here
            wsp = torch.zeros(max(L.llmq_awq_gemm_workspace_bytes(M, N, K), 16), dtype=torch.uint8, device=dev)

            def fn(it, a=(x, out, wsp, copies, M, N, K)):
                x_, out_, wsp_, copies_, M_, N_, K_ = a
                c = copies_[it % len(copies_)]
                rc = L.llmq_awq_gemm(x_.data_ptr(), K_, c[0].data_ptr(), c[2].data_ptr(), c[1].data_ptr(), None,
                                     out_.data_ptr(), M_, N_, K_, 128, wsp_.data_ptr(), wsp_.numel(), stream)
                assert rc == 0
            launches.append((f"{pname}_M{M}", M, N, K, fn))
    torch.cuda.synchronize()
    return launches


def roofline_w4a16(dev, passes):
    """AWQ W4A16 decode (M <= 16) of configs[3], weights streamed from HBM: sum of algorithmic bytes over the time of
    the 12 launches issued back to back in the order of `--awq-only` (which the tracked profiler summary traces, with
    the M = 64 launches in between).  These kernels last 7-25 us, less than a pair of event records costs when it
    brackets every launch, so one pair brackets each pass and the launch gaps are part of the figure."""
    from llmqrt_amd import workloads as W
    launches = awq_launch_set(dev, [m for m in W.AWQ_M if m <= 16])
    stream_obj = torch.cuda.current_stream()
    for it in range(3):
        for l in launches:
            l[4](it)
    torch.cuda.synchronize()
    pass_us = []
    for it in range(max(passes, 20)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream_obj)
        for l in launches:
            l[4](it + 3)
        e1.record(stream_obj)
        e1.synchronize()
        pass_us.append(e0.elapsed_time(e1) * 1e3)
    tot = statistics.median(pass_us)
    b = sum(W.awq_gemm_bytes(M, N, K) for _, M, N, K, _ in launches)
    ach = b / tot / 1e3
    return {"bound": "hbm", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(ach / PEAK_HBM_GBS, 4), "traffic": W4A16_TRAFFIC_BYTES,
            "algorithmic_bytes": b // len(launches),
            "kernel": "AWQ decode kernels behind llmq_awq_gemm at M in {1, 4, 16} x {qkv, o, gate_up, down}",
            "avg_launch_us": round(tot / len(launches), 2), "launches_per_pass": len(launches)}


def details_awq(dev, full=True):
    from llmqrt_amd import _abi, workloads as W
    L = _abi.lib()
    stream_obj = torch.cuda.current_stream()
    stream = stream_obj.cuda_stream
    rows = []
    for pi, (pname, (K, N)) in enumerate(W.QWEN2_7B_PROJ.items()):
        qw, qz, sc = W.awq_weights(N, K, W.seed_for(3, 100 + pi))
        wbytes = qw.numel() * 4 + qz.numel() * 4 + sc.numel() * 2
        ncopies = max(2, -(-320 * 1024 * 1024 // wbytes))  # rotate through > 256 MB (Infinity Cache) of weights
        copies = [(qw.to(dev).clone(), qz.to(dev).clone(), sc.to(dev).clone()) for _ in range(ncopies)]
        for mi, M in enumerate(W.AWQ_M):
            x = W.activations(M, K, W.seed_for(3, 10 * pi + mi), dtype=torch.float16, outliers=False).to(dev)
            out = torch.empty((M, N), dtype=torch.float16, device=dev)
            wsb = L.llmq_awq_gemm_workspace_bytes(M, N, K)
            wsp = torch.zeros(max(wsb, 16), dtype=torch.uint8, device=dev)  # arrival counters at its start: cleared once

            def mk(c):
                def f():
                    L.llmq_awq_gemm(x.data_ptr(), K, c[0].data_ptr(), c[2].data_ptr(), c[1].data_ptr(), None,
                                    out.data_ptr(), M, N, K, 128, wsp.data_ptr(), wsp.numel(), stream)
                return f
            fns = [mk(c) for c in copies]
            t_rot = batch_time_us(fns, stream_obj, max(2 * ncopies, 40))
            t_res = batch_time_us(fns[:1], stream_obj, 40)
            b = W.awq_gemm_bytes(M, N, K)
            rows.append({"proj": pname, "M": M, "us_hbm": round(t_rot, 2), "us_cache_resident": round(t_res, 2),
                         "GBs_hbm": round(b / t_rot / 1e3, 1), "pct_hbm_peak": round(100 * b / t_rot / 1e3 / PEAK_HBM_GBS, 2),
                         "GBs_cache_resident": round(b / t_res / 1e3, 1), "weight_copies_rotated": ncopies})
        if not full:
            del copies
            continue
        # prefill side of the module: the dequantizers (weights resident), alone and followed by this library's fp16
        # MFMA GEMM (the module's path above its token threshold); the vendor fp16 matmul on the [K, N] tensor is
        # timed beside it for context only
        deq = torch.empty((K, N), dtype=torch.float16, device=dev)
        deq_t = torch.empty((N, K), dtype=torch.float16, device=dev)
        c = copies[0]

        def dequant():
            L.llmq_awq_dequant(c[0].data_ptr(), c[2].data_ptr(), c[1].data_ptr(), deq.data_ptr(), K, N, 128, stream)

        def dequant_t():
            L.llmq_awq_dequant_t(c[0].data_ptr(), c[2].data_ptr(), c[1].data_ptr(), deq_t.data_ptr(), K, N, 128, stream)
        t_deq = batch_time_us([dequant], stream_obj, 40)
        t_deq_t = batch_time_us([dequant_t], stream_obj, 40)

        def own_path(xm, om, wsm):
            def f():
                dequant_t()
                L.llmq_gemm_f16(xm.data_ptr(), K, deq_t.data_ptr(), K, 1.0, None, 0, 0.0, om.data_ptr(), 1, N, xm.shape[0], N, K,
                                None, wsm.data_ptr(), wsm.numel(), stream)
            return f
        mid = {}
        for Mm in (256, 512, 2048):
            xm = W.activations(Mm, K, W.seed_for(3, 950 + pi + Mm), dtype=torch.float16, outliers=False).to(dev)
            om = torch.empty((Mm, N), dtype=torch.float16, device=dev)
            wsm = torch.empty(max(L.llmq_awq_gemm_workspace_bytes(Mm, N, K), L.llmq_gemm_f16_workspace_bytes(Mm, N, K), 16),
                              dtype=torch.uint8, device=dev)

            def fused():
                L.llmq_awq_gemm(xm.data_ptr(), K, c[0].data_ptr(), c[2].data_ptr(), c[1].data_ptr(), None, om.data_ptr(),
                                Mm, N, K, 128, wsm.data_ptr(), wsm.numel(), stream)

            def vendor():
                dequant()
                torch.matmul(xm, deq)
            mid[f"M{Mm}_tile_kernel_us"] = round(batch_time_us([fused], stream_obj, 10), 1)
            mid[f"M{Mm}_dequant_t_plus_gemm_f16_us"] = round(batch_time_us([own_path(xm, om, wsm)], stream_obj, 10), 1)
            mid[f"M{Mm}_dequant_plus_vendor_matmul_us"] = round(batch_time_us([vendor], stream_obj, 10), 1)
        db = K * N // 2 + 2 * K * N
        t_pre = mid["M2048_dequant_t_plus_gemm_f16_us"]
        rows.append({"proj": pname, **mid, "dequant_us": round(t_deq, 2), "dequant_GBs": round(db / t_deq / 1e3, 1),
                     "dequant_pct_hbm_peak": round(100 * db / t_deq / 1e3 / PEAK_HBM_GBS, 2),
                     "dequant_t_us": round(t_deq_t, 2), "dequant_t_GBs": round(db / t_deq_t / 1e3, 1),
                     "prefill_M2048_TFLOPs": round(2 * 2048 * N * K / t_pre / 1e6, 1)})
        del copies
    return rows


def awq_only(dev, steps, warmup):
    """For profiler runs: the launches of awq_launch_set (every token count of configs[3]) after one plain copy of
    known size that calibrates the HBM byte counters."""
    from llmqrt_amd import workloads as W
    cal_src = torch.zeros(64 << 20, dtype=torch.int32, device=dev)
    cal_dst = torch.empty_like(cal_src)
    cal_dst.copy_(cal_src)
    launches = awq_launch_set(dev, W.AWQ_M)
    for it in range(warmup + steps):
        for _, _, _, _, fn in launches:
            fn(it)
    torch.cuda.synchronize()
    print(json.dumps({"awq_only": True, "order": [l[0] for l in launches], "steps": steps, "warmup": warmup,
                      "calibration_copy_bytes_each_way": cal_src.numel() * 4}))


AWQ_PREFILL_M = (128, 256, 512, 2048)


def awq_prefill_only(dev, steps, warmup):
    """For profiler runs: the W4A16 tile kernel (more than 64 tokens) on the four projections, after one plain
    copy of known size that calibrates the HBM byte counters."""
    from llmqrt_amd import _abi, workloads as W
    L = _abi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    cal_src = torch.zeros(64 << 20, dtype=torch.int32, device=dev)
    cal_dst = torch.empty_like(cal_src)
    cal_dst.copy_(cal_src)
    launches, order = [], []
    for pi, (pname, (K, N)) in enumerate(W.QWEN2_7B_PROJ.items()):
        qw, qz, sc = (t.to(dev) for t in W.awq_weights(N, K, W.seed_for(3, 100 + pi)))
        for mi, M in enumerate(AWQ_PREFILL_M):
            x = W.activations(M, K, W.seed_for(3, 50 * pi + mi), dtype=torch.float16, outliers=False).to(dev)
            out = torch.empty((M, N), dtype=torch.float16, device=dev)
            wsp = torch.zeros(max(L.llmq_awq_gemm_workspace_bytes(M, N, K), 16), dtype=torch.uint8, device=dev)
            launches.append((x, out, wsp, (qw, qz, sc), M, N, K))
            order.append(f"{pname}_M{M}")
    torch.cuda.synchronize()
    for it in range(warmup + steps):
        for (x, out, wsp, c, M, N, K) in launches:
            rc = L.llmq_awq_gemm(x.data_ptr(), K, c[0].data_ptr(), c[2].data_ptr(), c[1].data_ptr(), None, out.data_ptr(),
                                 M, N, K, 128, wsp.data_ptr(), wsp.numel(), stream)
            assert rc == 0
    torch.cuda.synchronize()
    print(json.dumps({"awq_prefill_only": True, "order": order, "steps": steps, "warmup": warmup,
                      "calibration_copy_bytes_each_way": cal_src.numel() * 4}))


def quant_only(dev, steps, warmup):
    """For profiler runs: the HBM-bound row kernels in a fixed order after one calibration copy."""
    from llmqrt_amd import _abi, workloads as W
    L = _abi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    cal_src = torch.zeros(64 << 20, dtype=torch.int32, device=dev)
    cal_dst = torch.empty_like(cal_src)
    cal_dst.copy_(cal_src)
    cases, order = [], []
    for M in (2048, 8192):
        for K in (3584, 18944):
            x = W.activations(M, K, W.seed_for(1, 700 + M % 13 + K % 7)).to(dev)
            w = torch.ones(K, dtype=torch.bfloat16, device=dev)
            q = torch.empty((M, K), dtype=torch.int8, device=dev)
            y = torch.empty_like(x)
            sc = torch.empty(M, dtype=torch.float32, device=dev)
            cases.append((x, w, q, y, sc, M, K))
            order += [f"{k}_M{M}_K{K}" for k in ("quant_i8", "quant_fp8", "rmsnorm", "rmsnorm_quant_i8")]
    torch.cuda.synchronize()
    for _ in range(warmup + steps):
        for (x, w, q, y, sc, M, K) in cases:
            rc = L.llmq_quant_i8_per_token(x.data_ptr(), 0, M, K, K, q.data_ptr(), sc.data_ptr(), 2, stream)
            rc |= L.llmq_quant_fp8_per_token(x.data_ptr(), 0, M, K, K, q.data_ptr(), sc.data_ptr(), stream)
            rc |= L.llmq_rmsnorm(x.data_ptr(), 0, M, K, K, w.data_ptr(), 1e-6, y.data_ptr(), None, stream)
            rc |= L.llmq_rmsnorm_quant_i8_per_token(x.data_ptr(), 0, M, K, K, w.data_ptr(), 1e-6, None, q.data_ptr(),
                                                    sc.data_ptr(), 2, None, stream)
            assert rc == 0
    torch.cuda.synchronize()
    print(json.dumps({"quant_only": True, "order": order, "steps": steps, "warmup": warmup,
                      "calibration_copy_bytes_each_way": cal_src.numel() * 4}))


def details_layer(dev):
    """Config 4: one decoder layer's linears (qkv, o, gate_up, down) in W8A8 with SmoothQuant factors
    (alpha = 0.5) folded into the preceding RMSNorm weight (qkv, gate_up: one fused RMSNorm + per-token
    quantizer launch on the residual stream) or into the producer's weights (o, down: their inputs arrive
    divided by s; plain per-token quantizer); prefill 2048 tokens and decode 32.  The same tensors and launches
    are checked against the oracle in tests/test_gpu_layer_stack.py."""
    from llmqrt_amd import _abi, workloads as W
    stream_obj = torch.cuda.current_stream()
    stream = stream_obj.cuda_stream
    out = []
    layer = W.smoothquant_layer(alpha=0.5)
    dev_w = {n: (p["qweight"].to(dev), p["w_scale"].to(dev),
                 None if p["norm_weight_folded"] is None else p["norm_weight_folded"].to(dev))
             for n, p in layer.items()}
    for M in W.LAYER_M:
        lins = []
        for pname, p in layer.items():
            qw, scale, gf = dev_w[pname]
            lins.append(W8A8Linear(f"{pname}_M{M}", M, p["K"], p["N"], qw, scale, 0, dev,
                                   x=W.layer_input(pname, M, p["s"]), norm_weight=gf, eps=W.LAYER_NORM_EPS))

        def run_layer():
            for l in lins:
                l.launch(stream)
        t = batch_time_us([run_layer], stream_obj, 10)
        ops = sum(l.ops for l in lins)
        per = {}
        for l in lins:
            per[l.name] = round(batch_time_us([lambda l=l: l.launch(stream)], stream_obj, 10), 2)
        row = {"M": M, "layer_linear_us": round(t, 2), "TOPS": round(ops / t / 1e6, 1), "per_linear_us": per}
        if M <= 64:
            # decode is launch-bound: the same eight kernels captured once into a HIP graph and replayed
            # (the C ABI launches on the capturing stream and allocates nothing, so capture just works)
            side = torch.cuda.Stream()
            side.wait_stream(stream_obj)
            with torch.cuda.stream(side):
                s_side = side.cuda_stream
                for l in lins:
                    l.launch(s_side)
                side.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    for l in lins:
                        l.launch(torch.cuda.current_stream().cuda_stream)
            stream_obj.wait_stream(side)
            tg = batch_time_us([graph.replay], stream_obj, 10)
            row["layer_linear_us_hip_graph"] = round(tg, 2)
        out.append(row)
    return out


def details_few_tokens(dev):
    """W8A8 linears at 1 / 16 / 32 tokens with the weights coming out of HBM (rotated through > 256 MB of copies, as in
    a model whose weights do not fit the Infinity Cache): per-token quantizer + GEMM as two launches (the few-token
    GEMM kernel or the tile kernel, as the plan decides) against the one-launch linear that quantizes inside the GEMM
    kernel (where the token count fits it)."""
    from llmqrt_amd import _abi, workloads as W
    L = _abi.lib()
    stream_obj = torch.cuda.current_stream()
    stream = stream_obj.cuda_stream
    out = []
    for pi, (pname, (K, N)) in enumerate(W.QWEN2_7B_PROJ.items()):
        qw, ws = W.int8_weights(N, K, W.seed_for(1, 100 + pi))
        ncopies = max(2, -(-320 * 1024 * 1024 // (N * K)))
        copies = [qw.to(dev).clone() for _ in range(ncopies)]
        ws = ws.to(dev)
        row = {"proj": pname, "weight_MB": round(N * K / 1e6, 1)}
        for M in (1, 16, 32):
            x = W.activations(M, K, 7).to(dev)
            q = torch.empty((M, K), dtype=torch.int8, device=dev)
            sa = torch.empty(M, dtype=torch.float32, device=dev)
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
            nws = max(int(L.llmq_gemm_workspace_bytes(M, N, K)), 16)
            wsp = torch.empty(nws, dtype=torch.uint8, device=dev)

            def two(c):
                def f():
                    rc = L.llmq_quant_i8_per_token(x.data_ptr(), _abi.BF16, M, K, K, q.data_ptr(), sa.data_ptr(), _abi.F32, stream)
                    rc |= L.llmq_gemm_w8a8(q.data_ptr(), K, c.data_ptr(), K, sa.data_ptr(), ws.data_ptr(), 1.0, None, None, 0, 0.0,
                                           y.data_ptr(), _abi.BF16, N, M, N, K, None, wsp.data_ptr(), nws, stream)
                    return rc
                return f

            def one(c):
                return lambda: L.llmq_linear_i8_dynamic(x.data_ptr(), _abi.BF16, K, c.data_ptr(), K, ws.data_ptr(), None, 0,
                                                        y.data_ptr(), _abi.BF16, N, M, N, K, None, None, None, stream)
            assert two(copies[0])() == 0
            row[f"M{M}_quant_plus_gemm_us"] = round(batch_time_us([two(c) for c in copies], stream_obj, max(2 * ncopies, 40)), 2)
            if M <= L.llmq_linear_dynamic_max_tokens(K):
                assert one(copies[0])() == 0
                row[f"M{M}_one_launch_us"] = round(batch_time_us([one(c) for c in copies], stream_obj, max(2 * ncopies, 40)), 2)
        out.append(row)
        del copies
    return out


def details_norm_quant(dev):
    """RMSNorm feeding the per-token int8 quantizer: one fused kernel against the two separate ones."""
    from llmqrt_amd import _abi, workloads as W
    L = _abi.lib()
    stream_obj = torch.cuda.current_stream()
    stream = stream_obj.cuda_stream
    out = []
    K = 3584
    w = torch.ones(K, dtype=torch.bfloat16, device=dev)
    for M in (32, 2048, 8192):
        x = W.activations(M, K, W.seed_for(4, 300 + M % 97)).to(dev)
        y = torch.empty_like(x)
        q = torch.empty((M, K), dtype=torch.int8, device=dev)
        sc = torch.empty(M, dtype=torch.float32, device=dev)

        def fused():
            return L.llmq_rmsnorm_quant_i8_per_token(x.data_ptr(), 0, M, K, K, w.data_ptr(), 1e-6, None, q.data_ptr(),
                                                     sc.data_ptr(), 2, None, stream)

        def norm():
            return L.llmq_rmsnorm(x.data_ptr(), 0, M, K, K, w.data_ptr(), 1e-6, y.data_ptr(), None, stream)

        def quant():
            return L.llmq_quant_i8_per_token(y.data_ptr(), 0, M, K, K, q.data_ptr(), sc.data_ptr(), 2, stream)

        def two():
            norm()
            return quant()
        assert fused() == 0 and two() == 0
        tf = batch_time_us([fused], stream_obj, 20)
        tt = batch_time_us([two], stream_obj, 20)
        fused_bytes = 3 * M * K + 4 * M + 2 * K
        out.append({"M": M, "K": K, "fused_us": round(tf, 2), "norm_then_quant_us": round(tt, 2),
                    "fused_GBs": round(fused_bytes / tf / 1e3, 1),
                    "pct_hbm_peak": round(100 * fused_bytes / tf / 1e3 / PEAK_HBM_GBS, 2)})
    return out


def micro():
    """Microbenchmarks of the resources that bound the kernels (llmqrt_amd/csrc/microbench.hip); one JSON line."""
    import ctypes
    path = os.path.join(ROOT, "llmqrt_amd", "lib", "libllmq_microbench_gfx950.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: run `python -m llmqrt_amd.csrc.build`")
    mb = ctypes.CDLL(path)
    val = ctypes.c_double()

    def call(fn, *a):
        rc = fn(*[ctypes.c_int(v) for v in a], ctypes.byref(val))
        if rc != 0:
            raise RuntimeError(f"{fn.__name__}{a} failed with {rc}")
        return val.value

    out = {"micro": True, "mfma_TOPS": {}, "lds_bytes_per_ns_per_cu": {}, "direct_load_bytes_per_ns_per_cu": {},
           "empty_kernel_us": {}, "w4_stream_GBs": {}}
    for n in (1, 8, 32):
        out["empty_kernel_us"][f"eager_chain_of_{n}"] = round(call(mb.llmq_mb_launch, 0, n), 2)
        out["empty_kernel_us"][f"graph_replay_of_{n}"] = round(call(mb.llmq_mb_launch, 1, n), 2)
    for kind, name in enumerate(("int8_32x32x32", "fp8_32x32x64", "fp16_32x32x16")):
        for data, dn in enumerate(("random", "zero")):
            out["mfma_TOPS"][f"{name}_{dn}"] = round(call(mb.llmq_mb_mfma, kind, data), 1)
    for mode, name in enumerate(("ds_read_b128", "ds_write_b128", "global_load_lds_dwordx4")):
        out["lds_bytes_per_ns_per_cu"][name] = round(call(mb.llmq_mb_lds, mode), 1)
    for total_mb, where in ((128, "infinity_cache"), (512, "hbm")):
        for sharing in (1, 2, 4, 8, 32):
            out["direct_load_bytes_per_ns_per_cu"][f"{where}_{sharing}_blocks_per_line"] = round(call(mb.llmq_mb_share, sharing, total_mb), 1)
    # packed AWQ weights of the Qwen2-7B projections, [K, N/8] int32; rows_per_wave = K / (waves x K splits)
    for pname, K, N in (("qkv", 3584, 4608), ("gate_up", 3584, 37888), ("down", 18944, 3584)):
        for mode, mn in enumerate(("regs", "regs_lds_roundtrip", "load_to_lds")):
            for nw, rows in ((2, 64), (2, 128), (4, 128), (4, 448)):
                out["w4_stream_GBs"][f"{pname}_{mn}_{nw}w_{rows}rows"] = round(call(mb.llmq_mb_stream, mode, nw, rows, K, N), 0)
    print(json.dumps(out))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: the quantized-linear path has no multi-GPU part "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    from llmqrt_amd import _abi, workloads as W
    _abi.lib()
    stream_obj = torch.cuda.current_stream()
    stream = stream_obj.cuda_stream

    if args.micro:
        micro()
        return
    if args.awq_only:
        awq_only(dev, args.steps, args.warmup)
        return
    if args.awq_prefill_only:
        awq_prefill_only(dev, args.steps, args.warmup)
        return
    if args.quant_only:
        quant_only(dev, args.steps, args.warmup)
        return
    if args.fp8_only:
        fp8_only(dev, args.steps, args.warmup)
        return

    linears = build_w8a8_sweep(dev)
    total_ops = sum(l.ops for l in linears)
    prefill = [l for l in linears if l.M >= 2048]

    if args.roofline_only:
        # For profiler runs: only the dominant kernel's launches, preceded by one plain copy of known
        # size (256 MiB read + 256 MiB written) that calibrates the HBM byte counters.
        cal_src = torch.zeros(64 << 20, dtype=torch.int32, device=dev)
        cal_dst = torch.empty_like(cal_src)
        for l in prefill:
            l.quant(stream)
        torch.cuda.synchronize()
        cal_dst.copy_(cal_src)
        for _ in range(args.warmup):
            for l in prefill:
                l.gemm(stream)
        torch.cuda.synchronize()
        for _ in range(args.steps):
            for l in prefill:
                l.gemm(stream)
        torch.cuda.synchronize()
        print(json.dumps({"roofline_only": True, "launches_per_step": len(prefill), "steps": args.steps,
                          "calibration_copy_bytes_each_way": cal_src.numel() * 4}))
        return

    def step():
        rc = 0
        for l in linears:
            rc |= l.launch(stream)
        return rc

    for _ in range(args.warmup):
        if step() != 0:
            raise RuntimeError("a launch failed during warm-up")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    value = total_ops / (elapsed / args.steps) / 1e12

    # ---- roofline of the dominant kernel: the int8 MFMA GEMM launches at the prefill shapes ----
    # Same launch sequence as --roofline-only (the one the committed profiler summary covers): all
    # shapes back to back, every launch bracketed by HIP events on the launch stream, no host sync
    # inside a pass.
    shape_us = sequence_time_us([(l.name, (lambda it, l=l: l.gemm(stream))) for l in prefill], stream_obj, max(args.steps, 5))
    ops_sum, us_sum, alg_bytes, per_shape = 0, 0.0, 0, []
    for l in prefill:
        t_mean = shape_us[l.name]
        ops_sum += l.ops
        us_sum += t_mean
        alg_bytes += W.w8a8_gemm_bytes(l.M, l.N, l.K)
        per_shape.append({"shape": l.name, "us": round(t_mean, 2), "TOPS": round(l.ops / t_mean / 1e6, 1),
                          "pct_int8_mfma_peak": round(100 * l.ops / t_mean / 1e6 / PEAK_INT8_TOPS, 2)})
    achieved = ops_sum / us_sum / 1e6
    roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                "frac": round(achieved / PEAK_INT8_TOPS, 4), "traffic": ROOFLINE_TRAFFIC_BYTES,
                "algorithmic_bytes": alg_bytes // len(prefill),
                "kernel": "gemm_tile_kernel<int8> at M in {2048, 8192} x {qkv, o, gate_up, down}",
                "avg_launch_us": round(us_sum / len(prefill), 2), "launches": per_shape}

    result = {
        "metric": "W8A8/FP8 GEMM TOPS (% MFMA peak); W4A16 decode GB/s (% HBM peak), 1 GPU",
        "value": round(value, 2), "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "configs[1]: SmoothQuant W8A8 sweep, Qwen2-7B qkv/o/gate_up/down x M in "
                               "{1,16,128,2048,8192}, per-token int8 quantizer kernel + int8 MFMA GEMM with "
                               "per-token x per-channel epilogue, bf16 in/out; value = sum(2MNK) / step time",
                   "linears_per_step": len(linears), "ops_per_step": total_ops},
        "pct_int8_mfma_peak": round(100 * value / PEAK_INT8_TOPS, 2),
        "roofline": roofline,
    }

    if not args.no_details:
        w8 = []
        for l in sorted(linears, key=lambda l: (l.name.rsplit("_M", 1)[0], l.M)):
            tg = batch_time_us([lambda l=l: l.gemm(stream)], stream_obj, 20)
            tq = batch_time_us([lambda l=l: l.quant(stream)], stream_obj, 20)
            tops = l.ops / tg / 1e6
            w8.append({"shape": l.name, "gemm_us": round(tg, 2), "quant_us": round(tq, 2), "gemm_TOPS": round(tops, 1),
                       "pct_int8_mfma_peak": round(100 * tops / PEAK_INT8_TOPS, 2),
                       "gemm_GBs": round(W.w8a8_gemm_bytes(l.M, l.N, l.K) / tg / 1e3, 1),
                       "quant_GBs": round(W.quant_bytes(l.M, l.K) / tq / 1e3, 1)})
        result["details"] = {"w8a8": w8}

    if not args.no_cpu:
        cpu, parity = cpu_baseline_and_parity(linears, dev)
        result["cpu_baseline"] = cpu
        result["parity"] = parity
    else:
        result["cpu_baseline"] = None

    del linears, prefill
    torch.cuda.empty_cache()
    # the other two parts of the metric, each with its own roofline object inside the headline's `roofline`
    result["roofline"]["fp8"] = roofline_fp8(dev, max(args.steps, 5))
    torch.cuda.empty_cache()
    result["roofline"]["w4a16"] = roofline_w4a16(dev, max(args.steps, 5))
    torch.cuda.empty_cache()
    for part in ("fp8", "w4a16"):  # the same figures as flat scalars, for readers that keep only scalar fields
        for key in ("achieved", "frac", "avg_launch_us", "traffic"):
            result["roofline"][f"{part}_{key}"] = result["roofline"][part][key]
        result["roofline"][f"{part}_unit"] = result["roofline"][part]["unit"]
    result["pct_fp8_mfma_peak_prefill"] = round(100 * result["roofline"]["fp8"]["frac"], 2)
    result["pct_hbm_peak_w4a16_decode"] = round(100 * result["roofline"]["w4a16"]["frac"], 2)
    if not args.no_details:
        result["details"]["fp8"] = details_fp8(dev)          # one shape at a time, launches repeated (operands warm)
        result["details"]["awq_w4a16"] = details_awq(dev)
        result["details"]["layer_stack_w8a8"] = details_layer(dev)
        result["details"]["rmsnorm_quant_i8"] = details_norm_quant(dev)
        result["details"]["w8a8_few_tokens_weights_from_hbm"] = details_few_tokens(dev)

    print(json.dumps(result))


if __name__ == "__main__":
    main()
