import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# the package's modules are imported by bare name, as the reference's scripts import its layers
# (model/compressgnn/gcn.py:3-8): every test file finds them, run alone or with the others
PACKAGE = os.path.join(ROOT, "compressgnn_amd")
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.join(ROOT, "oracle", "_ref"), PACKAGE,
          os.path.join(PACKAGE, "layer"), os.path.join(PACKAGE, "loader"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs the HIP kernels)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
