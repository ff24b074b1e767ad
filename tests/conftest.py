import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs an MI355X (run with -m gpu on the GPU box)')


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason='no GPU in this process')
    for item in items:
        if 'gpu' in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _range_flag_isolation(request):
    """The range flag of the fixed-point states is process-wide and sticky: lower it before every GPU test, so that a
    test reports what its own launches did, and say so when a test leaves it up without having looked at it."""
    if 'gpu' not in request.keywords:
        yield
        return
    import torch
    if not torch.cuda.is_available():
        yield
        return
    import lava_dl_amd.slayer as slayer
    torch.cuda.synchronize()
    slayer.clear_range_flag()
    yield
    torch.cuda.synchronize()
    if slayer.clear_range_flag():
        import warnings
        warnings.warn(f'{request.node.nodeid} left the range flag of the 32-bit states raised')
