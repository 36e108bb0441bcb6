"""Runs the examples CLI's check mode (compiled kernels against the fp64 loop, through the
layer-shaped adapters) for all 14 recurrences, as `python tests/examples.py --op X --check-flex`
does in the reference."""
import pytest

from flex_rnn_amd import examples

import warm

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('op', examples.OPS)
def test_example_check_flex(op):
    print(f'case example {op}', flush=True)
    a = warm.EXAMPLE_ARGS
    examples.main(['--op', op, '--check-flex', '--batchsz', str(a['B']), '--seqlen', str(a['T']),
                   '--modeldim', str(a['D']), '--headsz', str(a['C'])])
