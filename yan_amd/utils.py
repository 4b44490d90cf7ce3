"""Parity metric and kernel timing shared by tests and benchmarks (reference: `yan/utils.py`)."""
import os
import sys

import torch


def calc_diff(x: torch.Tensor, y: torch.Tensor):
    """1 - 2<x,y> / (|x|^2 + |y|^2), evaluated in fp64 (reference: yan/utils.py:109-113).
    0 for identical tensors, 1 when one side is all zero, 2 for y == -x; sensitive to scale, unlike cosine."""
    x, y = x.double(), y.double()
    return 1 - 2 * (x * y).sum() / (x * x + y * y).sum()


def count_bytes(tensors) -> int:
    """Total storage of a (nested) tuple of tensors (reference: yan/utils.py:115-122)."""
    return sum(count_bytes(t) if isinstance(t, (tuple, list)) else t.numel() * t.element_size() for t in tensors)


class _Quiet:
    """Point file descriptors 1 and 2 at /dev/null for the duration of the block."""

    def __init__(self, active: bool) -> None:
        self.active = active

    def __enter__(self):
        if self.active:
            sys.stdout.flush(), sys.stderr.flush()
            self.null = os.open(os.devnull, os.O_WRONLY)
            self.saved = (os.dup(1), os.dup(2))
            os.dup2(self.null, 1), os.dup2(self.null, 2)
        return self

    def __exit__(self, *_):
        if self.active:
            sys.stdout.flush(), sys.stderr.flush()
            os.dup2(self.saved[0], 1), os.dup2(self.saved[1], 2)
            for fd in (*self.saved, self.null):
                os.close(fd)


_TIME_UNITS = (('ms', 1e-3), ('us', 1e-6), ('s', 1.0))


def _parse_time(text: str) -> float:
    for unit, scale in _TIME_UNITS:
        if text.endswith(unit):
            return float(text[:-len(unit)]) * scale
    raise ValueError(f'unrecognised profiler time {text!r}')


def bench_kineto(fn, kernel_names, num_tests: int = 30, suppress_kineto_output: bool = False,
                 trace_path: str = None, barrier_comm_profiling: bool = False, flush_l2: bool = False):
    """Mean device time, in seconds, of the kernels whose names contain `kernel_names` (a string or a tuple of
    strings) over `num_tests` calls of `fn`, taken from torch.profiler's device activity
    (reference: yan/utils.py:50-107). Each name must select exactly one profiler row. `flush_l2` writes a
    512 MB buffer before every call so inputs come from HBM, not from L2 / Infinity Cache.
    `barrier_comm_profiling` is accepted for signature compatibility; this build runs on one GPU and has no
    collective to align on."""
    external = bool(os.environ.get('YAN_NSYS_PROFILING') or os.environ.get('YAN_ROCPROF_PROFILING'))
    fn()        # first call may build or tune and print
    torch.cuda.synchronize()

    def run_all():
        for _ in range(num_tests):
            if flush_l2:
                torch.empty(512 << 18, dtype=torch.int, device='cuda').zero_()
            fn()

    if external:        # an outside profiler wraps the process: just run the work
        run_all(), run_all()
        torch.cuda.synchronize()
        return 1

    with _Quiet(suppress_kineto_output):
        schedule = torch.profiler.schedule(wait=0, warmup=1, active=1, repeat=1)
        with torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CUDA], schedule=schedule) as prof:
            for _ in range(2):
                run_all()
                torch.cuda.synchronize()
                prof.step()

    names = (kernel_names,) if isinstance(kernel_names, str) else tuple(kernel_names)
    assert all(isinstance(n, str) for n in names)
    rows = prof.key_averages().table(sort_by='cuda_time_total', max_name_column_width=300).split('\n')
    times = []
    for name in names:
        hits = [r for r in rows if name in r]
        assert len(hits) == 1, f'Errors of the kernel {name} in the profiling table: {rows}'
        times.append(_parse_time(hits[0].split()[-2]))
    if trace_path is not None:
        prof.export_chrome_trace(trace_path)
    return tuple(times) if isinstance(kernel_names, tuple) else times[0]
