"""Workspaces of the split-K launches the Python entry points make (the C library takes its workspace from the caller).

A split-K launch leaves partial sums and arrival counters in a workspace (`Gemm::run_split_k` in gemm/fp8_gemm.hpp): the
counters must be zero when a launch starts, are zero again when it has run to its end, and launches that share a workspace
must not overlap on the device. The reference's template leaves `split` to the caller's keys and has no such state
(`yan/jit_kernels/gemm.py:13-18`); this module is what keeps it out of the caller's sight:

* eager launches share one workspace per (device, stream): launches on one stream run one after the other. At most
  `MAX_EAGER_WORKSPACES` are kept; the oldest goes back to torch's allocator, which hands it out again in stream order;
* launches recorded into a graph get a workspace of their own per capture, made and zeroed inside the capture (the fill is
  a node of the graph: every replay starts from zero counters, whatever happened before), never shared with another
  capture or with eager launches, and kept for the life of the process: a graph may be replayed on any stream, at any time;
* a workspace whose last launch reported an error has its counters cleared before it is used again;
* `YAN_SPLIT_K=0` switches split-K off: the entry points then allocate nothing and keep no state between calls.
"""
import ctypes
import os
from typing import Callable, Dict, Hashable, Optional

import torch

# kSplitKCounterBytes and kSplitKWorkspaceBytes of gemm/scheduler.hpp: arrival counters, then the partial sums of the
# largest plan the heuristics make.
SPLIT_K_COUNTER_BYTES = 16 * 1024
SPLIT_K_WORKSPACE_BYTES = SPLIT_K_COUNTER_BYTES + 256 * 128 * 128 * 4
# what the entries allocate per workspace: the split-K workspace proper, then scratch for the chained quantiser + GEMM entry
# (codes and scales of the activations: gemm.CAST_SCRATCH_BYTES)
WORKSPACE_ALLOCATION_BYTES = SPLIT_K_WORKSPACE_BYTES + (4 << 20)
MAX_EAGER_WORKSPACES = 8


def split_k_enabled() -> bool:
    return os.getenv('YAN_SPLIT_K', '1') not in ('', '0')


class WorkspaceBook:
    """Which workspace a launch gets. `make()` returns a fresh workspace with zero counters, `clear(workspace)` puts the
    counters of an existing one back to zero; both act on the current stream. Pure bookkeeping otherwise."""

    def __init__(self, make: Callable[[], object], clear: Callable[[object], None], max_eager: int = MAX_EAGER_WORKSPACES):
        self.make, self.clear, self.max_eager = make, clear, max_eager
        self.eager: Dict[Hashable, object] = {}
        self.captures: Dict[Hashable, object] = {}
        self.suspect = set()

    def get(self, device: int, stream: int, capture: Optional[int] = None):
        """The workspace of a launch on `stream` of `device`; `capture` is the id of the capture the stream is recording
        into, None for an eager launch."""
        if capture is not None:
            key = (device, capture)
            workspace = self.captures.get(key)
            if workspace is None:
                workspace = self.captures[key] = self.make()
            return workspace
        key = (device, stream)
        workspace = self.eager.get(key)
        if workspace is None:
            while len(self.eager) >= self.max_eager:
                oldest = next(iter(self.eager))
                self.eager.pop(oldest)
                self.suspect.discard(oldest)
            workspace = self.eager[key] = self.make()
        elif key in self.suspect:
            self.clear(workspace)
        self.suspect.discard(key)
        return workspace

    def launch_failed(self, device: int, stream: int, capture: Optional[int] = None) -> None:
        """A launch on this workspace reported an error: its counters may not be zero. (A capture's workspace is zeroed
        by the graph itself at every replay.)"""
        if capture is None:
            self.suspect.add((device, stream))


def _make_workspace() -> torch.Tensor:
    workspace = torch.empty(WORKSPACE_ALLOCATION_BYTES, dtype=torch.uint8, device='cuda')
    workspace[:SPLIT_K_COUNTER_BYTES].zero_()         # a fill kernel: may be recorded into a graph
    return workspace


def _clear_workspace(workspace: torch.Tensor) -> None:
    workspace[:SPLIT_K_COUNTER_BYTES].zero_()


_book = WorkspaceBook(_make_workspace, _clear_workspace)
_hip = None


def _hip_runtime():
    """The HIP runtime this process has loaded (torch's), for the one query torch does not expose."""
    global _hip
    if _hip is None:
        path = 'libamdhip64.so'
        try:
            with open('/proc/self/maps') as maps:
                for line in maps:
                    if 'libamdhip64' in line:
                        path = line.split()[-1]
                        break
        except OSError:
            pass
        lib = ctypes.CDLL(path)
        lib.hipStreamGetCaptureInfo.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_ulonglong)]
        lib.hipStreamGetCaptureInfo.restype = ctypes.c_int
        _hip = lib
    return _hip


def capture_id(stream: int) -> Optional[int]:
    """The id of the capture `stream` (a bare handle) is recording into; None when it is not capturing. Raises when the
    runtime will not say."""
    status, ident = ctypes.c_int(0), ctypes.c_ulonglong(0)
    rc = _hip_runtime().hipStreamGetCaptureInfo(ctypes.c_void_p(stream), ctypes.byref(status), ctypes.byref(ident))
    if rc != 0:
        raise RuntimeError(f'hipStreamGetCaptureInfo failed with HIP error {rc}')
    return int(ident.value) if status.value == 1 else None         # hipStreamCaptureStatusActive


_is_capturing = getattr(torch._C, '_cuda_isCurrentStreamCapturing', None) or torch.cuda.is_current_stream_capturing
_last = (None, None)            # (token, workspace) of the latest eager launch: the usual next one


def split_k_workspace(device: torch.device, stream: int):
    """(workspace, token) for a split-K launch on `stream` (the bare handle of the current stream), or (None, None) when
    split-K is switched off. Hand `token` to `split_k_launch_failed` if the launch reports an error."""
    global _last
    if os.environ.get('YAN_SPLIT_K', '1') in ('', '0'):
        return None, None
    capture = capture_id(stream) if _is_capturing() else None
    index = device.index
    if index is None:
        index = torch.cuda.current_device()
    token = (index, stream, capture)
    if token == _last[0]:
        return _last[1], token
    workspace = _book.get(index, stream, capture)
    if capture is None:
        _last = (token, workspace)
    return workspace, token


def split_k_launch_failed(token) -> None:
    global _last
    _last = (None, None)
    _book.launch_failed(*token)
