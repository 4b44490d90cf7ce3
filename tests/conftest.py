import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
# JIT kernels are looked up in (and, when missing, compiled into) the in-tree cache, so that what was compiled
# ahead of time on a machine without a GPU is what runs on the machine with one.
os.environ.setdefault('YAN_CACHE_DIR', os.path.join(ROOT, '.yan_cache'))


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu)')


@pytest.fixture(scope='session')
def repo_root():
    return ROOT
