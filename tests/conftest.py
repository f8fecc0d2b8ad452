import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu)')


def pytest_collection_modifyitems(config, items):
    """GPU tests announce themselves before they start: a fault that ends the box still leaves the test's name behind"""
    for it in items:
        if it.get_closest_marker('gpu'):
            it.add_marker(pytest.mark.usefixtures('_announce'))


@pytest.fixture
def _announce(request):
    print(f'\n[gpu-case] {request.node.nodeid}', flush=True)
    yield
