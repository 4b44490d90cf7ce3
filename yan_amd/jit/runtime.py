"""Loaded JIT kernels: a cache directory holding `kernel.cu`, `kernel.args`, `kernel.so`, called through ctypes.

Contract of the reference's `yan/jit/runtime.py` (`Runtime` :13-68, `RuntimeCache` :71-86): a directory is a
valid kernel iff the three files exist; the library is opened lazily on first call; every call checks the
argument count and each argument's dtype/type against `kernel.args`, then calls `launch(*cargs, &rc)` and
returns `rc`. Work is enqueued on the stream that is passed in and is not synchronised here.
"""
import ctypes
import os
from typing import Dict, Optional

import torch

from .template import ctype_map

KERNEL_FILES = ('kernel.cu', 'kernel.args', 'kernel.so')


class Runtime:
    def __init__(self, path: str) -> None:
        self.path = path
        self.lib = None
        self.args = None
        self._launch = None
        assert self.is_path_valid(path), f'{path} is not a complete JIT kernel directory'

    @staticmethod
    def is_path_valid(path: str) -> bool:
        return os.path.isdir(path) and all(os.path.exists(os.path.join(path, f)) for f in KERNEL_FILES)

    def _load(self) -> None:
        self.lib = ctypes.CDLL(os.path.join(self.path, 'kernel.so'))
        self._launch = self.lib.launch
        self._launch.restype = None
        with open(os.path.join(self.path, 'kernel.args'), 'r') as f:
            # The file is a comma-joined list of ('name', type) tuples spelled with `torch` in scope.
            self.args = eval(f.read(), {'torch': torch, '__builtins__': {'bool': bool, 'int': int, 'float': float}})
        if self.args and not isinstance(self.args[0], tuple):
            self.args = (self.args,)      # a single ('name', type) pair evaluates to a flat tuple
        # Declared once so that ctypes marshals plain Python ints (device pointers, stream handles) and scalars itself.
        self._launch.argtypes = [ctype_map[dtype] for _, dtype in self.args] + [ctypes.POINTER(ctypes.c_int)]

    def __call__(self, *args) -> int:
        if self._launch is None:
            self._load()
        assert len(args) == len(self.args), f'Expected {len(self.args)} arguments, got {len(args)}'
        cargs = []
        for arg, (name, dtype) in zip(args, self.args):
            if isinstance(arg, torch.Tensor):
                assert arg.dtype == dtype, f'Expected tensor dtype `{dtype}` for `{name}`, got `{arg.dtype}`'
                cargs.append(arg.data_ptr())
            elif dtype is torch.cuda.Stream:
                # a Stream object, or its bare hipStream_t handle as an int (on ROCm `cuda_stream` is that handle)
                assert isinstance(arg, (torch.cuda.Stream, int)), f'Expected a stream for `{name}`, got `{type(arg)}`'
                cargs.append(arg if isinstance(arg, int) else arg.cuda_stream)
            else:
                assert isinstance(arg, dtype), f'Expected built-in type `{dtype}` for `{name}`, got `{type(arg)}`'
                cargs.append(arg)
        rc = ctypes.c_int(0)
        self._launch(*cargs, rc)
        return rc.value


class RuntimeCache:
    """In-process map path -> Runtime that falls back to whatever a previous process left on disk."""

    def __init__(self) -> None:
        self.cache: Dict[str, Runtime] = {}

    def __getitem__(self, path: str) -> Optional[Runtime]:
        hit = self.cache.get(path)
        if hit is None and Runtime.is_path_valid(path):
            hit = self.cache[path] = Runtime(path)
        return hit

    def __setitem__(self, path: str, runtime: Runtime) -> None:
        self.cache[path] = runtime
