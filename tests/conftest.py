import hashlib
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu)')


def pytest_addoption(parser):
    parser.addoption('--seed', type=int, default=0, help='base seed mixed into every test\'s RNG seed')


@pytest.fixture(autouse=True)
def seed(request):
    """Deterministic per-test seed: base seed + hash of the test id."""
    s = request.config.getoption('--seed') + int(hashlib.sha256(request.node.nodeid.encode()).hexdigest(), 16) % (2 ** 31)
    torch.manual_seed(s)
    return s


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason='no GPU in this process')
    for item in items:
        if 'gpu' in item.keywords:
            item.add_marker(skip)
