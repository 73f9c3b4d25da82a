"""Time the skinny GEMM the way the reference package does (operators/skinny_gemm/benchmarking_fn.py:8-101): a HIP
graph of `graph_size` calls, each on its own weight so that no call finds its weight in cache, replayed
`warmups + iterations` times on a side stream."""
from typing import Any, Dict, Optional, Tuple

import torch

from hf_rocm_kernels.utils.benchmarking import _time_graph_replays
from hf_rocm_kernels.utils.fp8 import amax_scale, fp8_quantize

from .binding import _skinny_gemm
from .wrapped import skinny_gemm


def benchmark_skinny_gemm(
    m: int,
    n: int,
    k: int,
    skg_kwargs: Optional[Dict[str, Any]] = None,
    graph_size: int = 8,
    warmups: int = 32,
    iterations: int = 128,
    device: str = "cuda",
    mode: str = "mean",
) -> Tuple[float, float]:
    """(mean or median, standard deviation) of the microseconds per call.
    skg_kwargs None: torch._scaled_mm (hipBLASLt) on the same operands; {}: `skinny_gemm`; otherwise the raw op
    with the given knob integers (validated like the reference's, otherwise advisory)."""
    if mode not in ("mean", "median"):
        raise ValueError(f"Invalid mode: {mode}")
    a = torch.randn((m, k), device=device)
    sa = amax_scale(a)
    a8 = fp8_quantize(a, sa)[0]
    weights, scales = [], []
    for _ in range(graph_size):
        w = torch.randn((n, k), device=device)
        sw = amax_scale(w)
        weights.append(fp8_quantize(w, sw)[0].t())
        scales.append(sw.reshape(1))
    combined = [(sa * sw).reshape(1).contiguous() for sw in scales]
    output = torch.zeros((m, n), device=device, dtype=torch.float16)
    sa1 = sa.reshape(1)

    if skg_kwargs is None:
        def fn(i: int) -> None:
            torch._scaled_mm(a8, weights[i], scale_a=sa1, scale_b=scales[i], out_dtype=torch.float16, out=output)
    elif not skg_kwargs:
        def fn(i: int) -> None:
            skinny_gemm(skinny_a=a8, b=weights[i], scale_tensor=combined[i], output=output)
    else:
        def fn(i: int) -> None:
            _skinny_gemm(A=a8, B=weights[i], scale_tensor=combined[i], D=output, **skg_kwargs)

    stream = torch.cuda.Stream(device)
    with torch.cuda.stream(stream):
        fn(0)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(graph_size):
                fn(i)
        torch.cuda.synchronize()
        ts = torch.tensor(_time_graph_replays(graph, graph_size, warmups, iterations))
    centre = ts.mean().item() if mode == "mean" else ts.median().item()
    return centre, ts.std().item()


def benchmark_skinny_gemm_general(
    m: int, n: int, k: int, split_k: int, A_producers: int = 0, B_producers: int = 0, consumers: int = 0, a_lanes: int = 0,
    b_lanes: int = 0, qsize: int = 0, op_m: int = 0, ops: int = 0, graph_size: int = 8, warmups: int = 32,
    iterations: int = 128, device: str = "cuda",
) -> Tuple[float, float]:
    """Same with the knobs spelled out; split_k == 0 times torch._scaled_mm (reference: benchmarking_fn.py:103-203)."""
    kwargs = None if split_k == 0 else dict(split_k=split_k, A_producers=A_producers, B_producers=B_producers,
                                            consumers=consumers, a_lanes=a_lanes, b_lanes=b_lanes, qsize=qsize,
                                            op_m=op_m, ops=ops)
    return benchmark_skinny_gemm(m, n, k, kwargs, graph_size, warmups, iterations, device)
