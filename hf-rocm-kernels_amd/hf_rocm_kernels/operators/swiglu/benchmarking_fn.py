"""Time the SwiGLU operator the way the reference package does (operators/swiglu/benchmarking_fn.py:4-70)."""
import torch

from hf_rocm_kernels.utils.benchmarking import _time_graph_replays

from .reference import reference_swiglu
from .wrapped import swiglu


def benchmark_swiglu(
    batch_size: int,
    intermediate_size: int,
    num_threads: int,
    force_scalar: bool = False,
    graph_size: int = 16,
    warmups: int = 50,
    iterations: int = 250,
    device: str = "cuda",
) -> float:
    """Mean microseconds per call; num_threads 0 times the torch reference, -1 lets the launcher choose, a positive
    value is passed to the kernel."""
    inputs = [torch.randn((batch_size, 2 * intermediate_size), device=device).to(torch.float16) for _ in range(graph_size)]
    scales = [torch.rand((1,), device=device).mul(2).add(1) for _ in range(graph_size)]
    if num_threads == 0:
        def fn(i: int) -> None:
            reference_swiglu(inputs[i], scales[i])
    else:
        def fn(i: int) -> None:
            swiglu(inputs[i], scales[i], force_scalar=force_scalar, num_threads=num_threads)
    stream = torch.cuda.Stream(device)
    with torch.cuda.stream(stream):
        fn(0)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(graph_size):
                fn(i)
        torch.cuda.synchronize()
        samples = _time_graph_replays(graph, graph_size, warmups, iterations)
    return sum(samples) / len(samples)
