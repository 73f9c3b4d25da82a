"""Timing helpers with the names of the reference package's utils/benchmarking.py:9-135, built on HIP graphs and
HIP events only (the reference leans on triton's do_bench, which this package does not depend on).

Everything here times device work: a function is captured into a graph of `graph_size` calls and the graph is
replayed, so Python and launch overhead stay out of the figure.
"""
import itertools
import warnings
from typing import Any, Callable, Dict, Sequence

import torch


def randomize_tensors(x: Any) -> Any:
    """A fresh tensor of the same shape and dtype filled with N(0,1) draws (cast through fp32); anything that is
    not a tensor is returned as is."""
    if isinstance(x, torch.Tensor):
        return torch.randn(x.shape, device=x.device, dtype=torch.float32).to(x.dtype)
    return x


def _time_graph_replays(graph: "torch.cuda.CUDAGraph", calls: int, warmups: int, iterations: int,
                        between: Callable[[], None] = lambda: None) -> Sequence[float]:
    """Microseconds per call for each of `iterations` timed replays (after `warmups` untimed ones)."""
    samples = []
    for i in range(warmups + iterations):
        between()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        graph.replay()
        end.record()
        end.synchronize()
        if i >= warmups:
            samples.append(start.elapsed_time(end) * 1e3 / calls)
    return samples


def benchmark_cuda_graph_no_cache(fn: Callable, args: Sequence[Any], kwargs: Dict[str, Any], graph_size: int = 8,
                                  warmups: int = 32, iterations: int = 128, device: str = "cuda") -> float:
    """Mean microseconds per call of fn(*args, **kwargs), every call of the graph on its own randomised copy of
    the tensor arguments so that consecutive calls do not find their operands in cache."""
    arg_sets = [tuple(randomize_tensors(a) for a in args) for _ in range(graph_size)]
    kwarg_sets = [{k: randomize_tensors(v) for k, v in kwargs.items()} for _ in range(graph_size)]
    stream = torch.cuda.Stream(device)
    with torch.cuda.stream(stream):
        fn(*arg_sets[0], **kwarg_sets[0])  # outside capture: loads code, lets the op set up its workspace
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for a, kw in zip(arg_sets, kwarg_sets):
                fn(*a, **kw)
        torch.cuda.synchronize()
        samples = _time_graph_replays(graph, graph_size, warmups, iterations)
    return sum(samples) / len(samples)


class Bench:
    """Collects timings of several versions of one operator into a table: columns = versions, rows = labels."""

    def __init__(self) -> None:
        self.enter_benchmark_mode()
        self.check_device_is_free(warn_if_not=True)
        self._measures: Dict[str, Dict[Any, float]] = {}

    @classmethod
    def enter_benchmark_mode(cls, enable_tunable: bool = False) -> None:
        """No autograd bookkeeping while timing; optionally torch's TunableOp for the torch baselines."""
        torch.set_grad_enabled(False)
        if enable_tunable:
            torch.cuda.tunable.enable(val=True)

    def check_device_is_free(self, warn_if_not: bool = False) -> Dict[str, int]:
        """Memory already in use on the current device (a busy device distorts timings)."""
        free, total = torch.cuda.mem_get_info()
        metrics = {"memory_used_mb": int((total - free) >> 20), "memory_total_mb": int(total >> 20)}
        if warn_if_not and metrics["memory_used_mb"] > 2048:
            warnings.warn(f"Device {torch.cuda.current_device()} is not free: {metrics = }")
        return metrics

    @classmethod
    def benchmark_fn(cls, fn: Callable[[], None], rep: int = 100, warmup: int = 10, graph_size: int = 0) -> float:
        """Median microseconds per call of fn() from `rep` replays of a graph of `graph_size` calls.
        graph_size 0 sizes the graph from a first estimate so that one replay lasts about a millisecond (8 to 256
        calls): launching a graph costs some ten microseconds however small it is, which a graph of a few
        microsecond-sized kernels would otherwise report as kernel time (the reference gets the same effect from
        triton's do_bench_cudagraph, utils/benchmarking.py:60-75)."""
        stream = torch.cuda.Stream()

        def capture(calls: int) -> "torch.cuda.CUDAGraph":
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for _ in range(calls):
                    fn()
            torch.cuda.synchronize()
            return graph

        with torch.cuda.stream(stream):
            fn()
            torch.cuda.synchronize()
            if graph_size <= 0:
                probe = sorted(_time_graph_replays(capture(8), 8, 2, 5))
                graph_size = int(min(256, max(8, 1000.0 / max(probe[len(probe) // 2], 1e-3))))
            samples = sorted(_time_graph_replays(capture(graph_size), graph_size, max(warmup, 0), rep))
        return samples[len(samples) // 2]

    def add_measure(self, header: str, label: Any, fn: Callable[[], None], rep: int = 100) -> None:
        self.add_raw_measure(header, label, self.benchmark_fn(fn, rep))

    def add_raw_measure(self, header: str, label: Any, measure: float) -> None:
        """Put `measure` into column `header`, row `label`."""
        self._measures.setdefault(header, {})[label] = measure

    def add_speedup_column(self, ref_header: str, our_header: str) -> None:
        """Column "Speedup" = ref / ours for every row of the reference column."""
        if ref_header not in self._measures or our_header not in self._measures:
            raise ValueError(f"Headers {ref_header} and {our_header} must be present in the benchmark table.")
        for label, ref in self._measures[ref_header].items():
            if label in self._measures[our_header]:
                self.add_raw_measure("Speedup", label, ref / self._measures[our_header][label])

    def table(self, row_header: str) -> Dict[str, list]:
        rows = sorted(set(itertools.chain.from_iterable(m.keys() for m in self._measures.values())))
        data: Dict[str, list] = {row_header: rows}
        for header, measures in self._measures.items():
            data[header] = [measures.get(row, "-") for row in rows]
        return data

    def display_table(self, row_header: str) -> None:
        data = self.table(row_header)
        try:
            import tabulate
            print(tabulate.tabulate(data, list(data.keys())))
        except ImportError:
            print("\t".join(data.keys()))
            for i in range(len(data[row_header])):
                print("\t".join(str(col[i]) for col in data.values()))
