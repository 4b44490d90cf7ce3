"""Build-and-pick for JIT kernels.

Behaviour of the reference's `JITTuner.compile_and_tune` (`yan/jit_kernels/tuner.py:12-78`):

* results are memoised per `(name, sorted keys)`; the steady-state cost of a GEMM call is this dict lookup;
* every candidate in `space` is merged over `keys`, generated and built (a failing build raises);
* with more than one candidate each is run once (non-zero return code => the candidate is illegal and is
  skipped) and then timed over 20 back-to-back launches bracketed by device events, after a cache flush and
  a large matmul that absorbs launch jitter; the fastest wins;
* an empty `space` means "build exactly `keys`" and nothing is timed.
"""
import os
from typing import Any, Dict, Tuple

import torch

from ..jit import build, cpp_format, generate, Runtime

# MI355X keeps 256 MB of Infinity Cache behind the 8 L2s; writing this many bytes evicts a kernel's inputs.
FLUSH_BYTES = 512 << 20
TIMED_LAUNCHES = 20


def _time_candidate(runtime: Runtime, args: tuple) -> float:
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.empty(FLUSH_BYTES // 4, dtype=torch.int, device='cuda').zero_()
    lhs = torch.randn((4096, 4096), dtype=torch.float, device='cuda')
    lhs @ lhs
    start.record()
    for _ in range(TIMED_LAUNCHES):
        assert runtime(*args) == 0
    end.record()
    end.synchronize()
    return start.elapsed_time(end)


class FrozenKeys(dict):
    """Keys of a kernel plan that its owner promises never to change (the entry points memoise their plans and hand
    the same object over on every call): any attempt to modify one raises."""

    def _frozen(self, *_, **__):
        raise TypeError('the keys of a memoised kernel plan are read-only')

    __setitem__ = __delitem__ = clear = pop = popitem = setdefault = update = __ior__ = _frozen


class JITTuner:
    def __init__(self) -> None:
        self.tuned: Dict[Tuple[str, str], Runtime] = {}
        self.tuned_keys: Dict[Tuple[str, str], Dict[str, Any]] = {}
        # Callers that pass the very same FrozenKeys object again skip building the textual signature:
        # (name, id(keys)) -> (keys, runtime); the stored reference both keeps the id from being reused and is compared
        # on lookup. An ordinary dict, which its owner may change between calls, always takes the signature path, as
        # in the reference.
        self._same_object: Dict[Tuple[str, int], Tuple[Dict[str, Any], Runtime]] = {}

    def _remember(self, name: str, keys: Dict[str, Any], runtime: Runtime) -> None:
        if isinstance(keys, FrozenKeys):
            self._same_object[(name, id(keys))] = (keys, runtime)

    def compile_and_tune(self, name: str, keys: Dict[str, Any], space: tuple,
                         includes: tuple, arg_defs: tuple, template: str, args: tuple) -> Runtime:
        seen = self._same_object.get((name, id(keys)))
        if seen is not None and seen[0] is keys:
            return seen[1]
        caller_keys = keys
        keys = {k: keys[k] for k in sorted(keys)}
        signature = (name, str(keys))
        debug = bool(os.getenv('YAN_JIT_DEBUG'))
        hit = self.tuned.get(signature)
        if hit is not None:
            if debug:
                print(f'Using cached JIT kernel {name} with keys {keys}')
            self._remember(name, caller_keys, hit)
            return hit
        if debug:
            print(f'Auto-tuning JIT kernel {name} with keys {keys}')
        assert args is not None

        candidates = tuple(space) if len(space) > 0 else ({},)
        built = []
        for extra in candidates:
            assert isinstance(extra, dict)
            code = generate(includes, arg_defs, cpp_format(template, {**keys, **extra}))
            built.append((build(name, arg_defs, code), extra))     # an illegal build raises

        best = None     # (time, runtime, extra)
        for runtime, extra in built:
            elapsed = 0.0
            if len(candidates) > 1:
                rc = runtime(*args)
                if rc != 0:     # e.g. the tile does not fit LDS: not a candidate
                    if debug:
                        print(f'Illegal JIT kernel {name} with keys {keys} and tuned keys {extra}: error code {rc}')
                    continue
                elapsed = _time_candidate(runtime, args)
            if debug:
                print(f'Tuned JIT kernel {name} with keys {keys} and tuned keys {extra} has time {elapsed}')
            if best is None or elapsed < best[0]:
                best = (elapsed, runtime, extra)
        assert best is not None, f'Failed to tune JIT kernel {name} with keys {keys}'

        if debug or os.getenv('YAN_PRINT_AUTOTUNE'):
            print(f'Best JIT kernel {name} with keys {keys} has tuned keys {best[2]} and time {best[0]}')
        self.tuned[signature] = best[1]
        self.tuned_keys[signature] = dict(best[2])
        self._remember(name, caller_keys, best[1])
        return best[1]


jit_tuner = JITTuner()
