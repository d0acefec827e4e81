import os
import sys

import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
for path in (HERE, ROOT):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) GPU")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


from bench_workloads import rel_l2, seeded_bf16  # noqa: E402,F401  (tests import them from here)


@pytest.fixture
def gpu_division_rule():
    """Library and oracle both evaluate clamp(amax) / 448 the way ATen's GPU kernel does (product with fp32(1/448))
    for the duration of a test; the default (the correctly rounded quotient) is restored afterwards."""
    import lingua_amd
    import oracle
    lingua_amd.set_scale_rule("times_inverse")
    try:
        with oracle.scale_rule("times_inverse"):
            yield
    finally:
        lingua_amd.set_scale_rule("divide")
