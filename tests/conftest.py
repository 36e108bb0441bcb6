import os
import sys

import pytest

# every launch the tests make is audited first (tensor shapes, element types and storage bounds against what the
# kernel indexes; grid against the plan): read by flex_rnn_amd.launch when it is imported
os.environ.setdefault('FLEX_RNN_CHECK', '1')

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu)')


@pytest.fixture(scope='session')
def runtime_lib():
    """The in-tree C-ABI runtime; built once if a CPU-only run finds it missing."""
    from flex_rnn_amd import runtime
    if not os.path.isfile(runtime.LIB_PATH):
        runtime.build_library()
    return runtime.lib()
