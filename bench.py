"""Headline benchmark: FP8 skinny GEMM on Llama-3-8B decode linear shapes, one MI355X.

A step is one pass over BASELINE's second configuration: M in {1, 2, 4, 8, 16} x the four projection shapes
qkv (6144, 4096), o_proj (4096, 4096), gate_up (28672, 4096), down (4096, 14336) -- 20 calls of
`hf_rocm_kernels.skinny_gemm` (FP8 e4m3fn activations and weights, per-tensor scales, bf16 output accumulated
into a zeroed buffer, as the reference's callers do).  All inputs are resident in HBM before the clock starts.
Every call of a step reads a different copy of its weight, and a copy is read again only after ~1.5 GB of other
weights have been streamed, so nothing is served from the 256 MB Infinity Cache or from L2.

The calls of a step are captured once into a HIP graph (the reference times its kernel the same way,
operators/skinny_gemm/benchmarking_fn.py:62-92) so the figure is the GPU's, not the Python launch path's.

value       = algorithmic bytes of a step / time of a step, in GB/s (N*K + M*K + 2*M*N + 4 bytes per call)
roofline    = the same bytes over the same HIP-event time, against 8 TB/s of HBM3E
cpu_baseline= the oracle's torch path (dequantise -> fp32 matmul -> scale -> bf16) on the host cores, same shapes

traffic     = HBM bytes per launch read back from rocprofv3 counters (FETCH_SIZE and WRITE_SIZE runs of this
              script with `--copy-calibration`, which appends a plain 256 MiB device copy whose counter reading
              fixes the scale); the figure is a constant below because a benchmark cannot profile itself

Prints one JSON line.  `--detail` adds a per-(shape, M) table measured outside the timed region.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "hf-rocm-kernels_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

SHAPES = [("qkv", 6144, 4096), ("o_proj", 4096, 4096), ("gate_up", 28672, 4096), ("down", 4096, 14336)]
MS = [1, 2, 4, 8, 16]
HBM_PEAK_GBPS = 8000.0
# Mean HBM bytes per GEMM launch of a step (fetched + written), from the FETCH_SIZE / WRITE_SIZE counter runs
# summarised in profiles/skinny_gemm_stream_llama3_8b_decode_hbm_traffic.txt: 1.0096 x the algorithmic bytes.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = 55223910
CALIBRATION_COPY_BYTES = 256 << 20
WORKLOAD = ("llama3-8b decode linears: M in {1,2,4,8,16} x qkv(6144,4096) o_proj(4096,4096) gate_up(28672,4096) "
            "down(4096,14336); FP8 e4m3fn A and W, per-tensor scales, bf16 out; 20 calls per step")


def algorithmic_bytes(m, n, k):
    return n * k + m * k + 2 * m * n + 4


def make_inputs(torch, cycle):
    """Activations per M, and 5*cycle quantised copies of each weight, all on the GPU."""
    from hf_rocm_kernels.utils.fp8 import amax_scale, fp8_quantize
    gen = torch.Generator(device="cuda").manual_seed(0)
    acts, weights = {}, {}
    for m in MS:
        for _, n, k in SHAPES:
            if (m, k) in acts:
                continue
            a = torch.randn((m, k), generator=gen, device="cuda").to(torch.bfloat16).float()
            sa = amax_scale(a)
            acts[(m, k)] = (fp8_quantize(a, sa)[0], sa.reshape(1))
    for name, n, k in SHAPES:
        copies = []
        for _ in range(len(MS) * cycle):
            w = torch.randn((n, k), generator=gen, device="cuda").mul_(0.02)
            sw = amax_scale(w)
            copies.append((fp8_quantize(w, sw)[0].t(), sw.reshape(1)))
            del w
        weights[name] = copies
    return acts, weights


def capture_steps(torch, acts, weights, cycle):
    """One HIP graph per step of the rotation; step i uses weight copy i*5 + (index of M)."""
    import hf_rocm_kernels
    outs = {(m, n): torch.zeros((m, n), dtype=torch.bfloat16, device="cuda") for m in MS for _, n, _ in SHAPES}
    scales = {}
    for name, n, k in SHAPES:
        for ci, (w, sw) in enumerate(weights[name]):
            for m in MS:
                scales[(name, ci, m)] = (acts[(m, k)][1] * sw).contiguous()

    def run_step(i):
        for name, n, k in SHAPES:
            for mi, m in enumerate(MS):
                ci = i * len(MS) + mi
                w, _ = weights[name][ci]
                out = outs[(m, n)]  # the op accumulates into it; zeroing belongs to the producer of the buffer
                hf_rocm_kernels.skinny_gemm(acts[(m, k)][0], w, scales[(name, ci, m)], out)

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        run_step(0)  # warm-up outside capture: loads code objects, allocates the split-K workspace
    torch.cuda.synchronize()
    graphs = []
    for i in range(cycle):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            run_step(i)
        graphs.append(g)
    return graphs, outs


def time_cases(torch, acts, weights, cycle, reps=40):
    """Per-(shape, M) time from a graph of `5*cycle` calls over all copies of the weight, replayed `reps` times."""
    import hf_rocm_kernels
    rows = []
    stream = torch.cuda.Stream()
    for name, n, k in SHAPES:
        for m in MS:
            out = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
            a, sa = acts[(m, k)]
            sc = [(sa * sw).contiguous() for _, sw in weights[name]]
            with torch.cuda.stream(stream):
                hf_rocm_kernels.skinny_gemm(a, weights[name][0][0], sc[0], out)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for ci, (w, _) in enumerate(weights[name]):
                    hf_rocm_kernels.skinny_gemm(a, w, sc[ci], out)
            calls = len(weights[name])
            for _ in range(3):
                g.replay()
            torch.cuda.synchronize()
            ts = []
            for _ in range(reps):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                g.replay()
                e1.record()
                e1.synchronize()
                ts.append(e0.elapsed_time(e1) * 1e3 / calls)
            ts.sort()
            us = ts[len(ts) // 2]
            gbps = algorithmic_bytes(m, n, k) / us / 1e3
            rows.append({"shape": name, "n": n, "k": k, "m": m, "us_per_call": round(us, 3),
                         "us_std": round(float(torch.tensor(ts).std()), 3), "gbps": round(gbps, 1),
                         "frac_of_peak": round(gbps / HBM_PEAK_GBPS, 4)})
            del g
    return rows


def cpu_baseline(torch, budget_s=20.0):
    """The oracle's reference path on the host: one pass over the same 20 (shape, M) cases, repeated while the
    budget lasts (at least twice); median pass time.  Inputs are drawn on the CPU with the same recipe."""
    from oracle import fp8 as ofp8
    from oracle import skinny_gemm as og
    torch.set_num_threads(max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1))))
    gen = torch.Generator().manual_seed(0)
    cases = []
    for name, n, k in SHAPES:
        w = torch.randn((n, k), generator=gen) * 0.02
        sw = ofp8.amax_scale(w)
        w8 = ofp8.fp8_quantize(w, sw)[0].t()
        for m in MS:
            a = torch.randn((m, k), generator=gen).to(torch.bfloat16).float()
            sa = ofp8.amax_scale(a)
            cases.append((ofp8.fp8_quantize(a, sa)[0], w8, sa.reshape(1), sw.reshape(1), algorithmic_bytes(m, n, k)))
    total_bytes = sum(c[4] for c in cases)

    def one_pass():
        t0 = time.perf_counter()
        for a8, w8, sa, sw, _ in cases:
            og.reference_skinny_gemm(a8, w8, sa, sw)
        return time.perf_counter() - t0

    one_pass()  # warm-up
    times, spent = [], 0.0
    while len(times) < 2 or (spent < budget_s and len(times) < 9):
        t = one_pass()
        times.append(t)
        spent += t
    times.sort()
    med = times[len(times) // 2]
    return {"value": round(total_bytes / med / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "%d full passes over the same 20 (shape, M) cases, median pass %.3f s; oracle torch path "
                      "dequantise->fp32 matmul->scale->bf16" % (len(times), med),
            "ms_per_step": round(med * 1e3, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=140)
    ap.add_argument("--warmup", type=int, default=28)
    ap.add_argument("--detail", action="store_true", help="also time every (shape, M) case on its own")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-budget", type=float, default=20.0)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="after the timed steps run a plain device copy of known size (for scaling rocprofv3 byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the kernels have no CPU path)")
    torch.cuda.set_device(0)

    cycle = 7  # 35 copies of each weight: 7.6 GB in all, a copy is re-read after ~1.5 GB of other weights
    acts, weights = make_inputs(torch, cycle)
    graphs, outs = capture_steps(torch, acts, weights, cycle)
    step_bytes = sum(algorithmic_bytes(m, n, k) for _, n, k in SHAPES for m in MS)

    for i in range(args.warmup):
        graphs[i % cycle].replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(args.steps):
        graphs[i % cycle].replay()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    gpu_ms = e0.elapsed_time(e1)
    ms_per_step = gpu_ms / args.steps
    gbps = step_bytes / (ms_per_step * 1e-3) / 1e9
    calls = len(SHAPES) * len(MS)

    result = {
        "metric": "FP8 skinny-GEMM achieved HBM GB/s over Llama-3-8B decode shapes, M=1..16 (us/call in `cases`)",
        "value": round(gbps, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn",
        "data": "synthetic",
        "config": {"workload": WORKLOAD, "calls_per_step": calls, "bytes_per_step": step_bytes,
                   "weight_copies_per_shape": len(MS) * cycle, "timing": "HIP graph replay, HIP events",
                   "us_per_call_mean": round(ms_per_step * 1e3 / calls, 3), "wall_ms_per_step": round(wall_ms / args.steps, 5)},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH,
                     "kernel": "hfrk::skinny_gemm_stream_kernel<MA> (all 20 launches of a step)",
                     "bytes_per_launch": round(step_bytes / calls), "us_per_launch": round(ms_per_step * 1e3 / calls, 3)},
    }
    if args.copy_calibration:
        # bitwise_not over int32: one elementwise kernel that reads and writes CALIBRATION_COPY_BYTES each
        src = torch.arange(CALIBRATION_COPY_BYTES // 4, dtype=torch.int32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.bitwise_not(src, out=dst)
        torch.cuda.synchronize()
        result["config"]["calibration_copy_bytes"] = CALIBRATION_COPY_BYTES
        del src, dst
    if args.detail:
        result["cases"] = time_cases(torch, acts, weights, cycle)
    del graphs, weights, acts, outs
    torch.cuda.empty_cache()
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, args.cpu_budget)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
