import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


# Every network of the test session fills the LDS of all CUs with NaN patterns in front of each layer (a debugging aid
# of the library): the LDS keeps its contents between kernels, so a kernel that multiplies a location it never staged
# with a zero weight passes or fails by what ran before it unless the leftovers are made poisonous.
os.environ.setdefault("FYNHIP_POISON_LDS", "1")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def _gpu_present():
    return os.path.exists("/dev/kfd")


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU in this container (/dev/kfd missing)")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
