"""CPU restatement of the GEMM hot path. TEST INFRASTRUCTURE ONLY: nothing under `yan_amd/` imports this package;
it is used by `tests/`, by `__graft_entry__.smoke()` and by the `cpu_baseline` leg of `bench.py` as the checker."""
from .gemm_oracle import *  # noqa: F401,F403
