"""Skinny GEMM through its wrapper against torch._scaled_mm (hipBLASLt) on the same operands, one line per shape.

Counterpart of the reference package's benchmarks/skinny_gemm/no_knobs.py:20-52.  Usage, from the repository root:
    python hf-rocm-kernels_amd/hf_rocm_kernels/benchmarks/skinny_gemm/no_knobs.py -m 1 8 16 -n 4096 28672 -k 4096
Every call of a timed graph reads its own weight, so weights come from HBM, not from cache.
"""
import argparse
import itertools
import os
import sys

if __package__ in (None, ""):
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "..", ".."))

from hf_rocm_kernels.operators.skinny_gemm.benchmarking_fn import benchmark_skinny_gemm  # noqa: E402


def main() -> None:
    parser = argparse.ArgumentParser()
    parser.add_argument("--m", "-m", type=int, nargs="+", default=[1, 8, 16])
    parser.add_argument("--n", "-n", type=int, nargs="+", default=[4096])
    parser.add_argument("--k", "-k", type=int, nargs="+", default=[4096])
    parser.add_argument("--graph-size", type=int, default=16)
    parser.add_argument("--warmups", type=int, default=50)
    parser.add_argument("--iterations", type=int, default=200)
    parser.add_argument("--device", default="cuda:0")
    args = parser.parse_args()
    print(f"{'m':>4} {'n':>6} {'k':>6} {'_scaled_mm us':>16} {'skinny_gemm us':>16} {'speedup':>8} {'GB/s':>8}")
    for m, n, k in itertools.product(args.m, args.n, args.k):
        common = dict(graph_size=args.graph_size, warmups=args.warmups, iterations=args.iterations, device=args.device,
                      mode="median")
        try:
            t_ref, s_ref = benchmark_skinny_gemm(m, n, k, None, **common)
        except Exception as e:  # a torch build without the fp8 hipBLASLt path
            t_ref, s_ref = float("nan"), 0.0
            print(f"# torch._scaled_mm unavailable: {e}")
        t, s = benchmark_skinny_gemm(m, n, k, {}, **common)
        gbps = (n * k + m * k + 2 * m * n) / t / 1e3
        print(f"{m:4d} {n:6d} {k:6d} {t_ref:9.2f} ±{s_ref:5.2f} {t:9.2f} ±{s:5.2f} {t_ref / t:8.2f} {gbps:8.0f}")


if __name__ == "__main__":
    main()
