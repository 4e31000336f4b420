import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; run with -m gpu")


def pytest_report_header(config):
    """Which native libraries the tests will load, and whether they were built from the sources beside them."""
    from mini_gpt_inference_amd.csrc import build

    lines = []
    for path, files, flags in ((build.kernel_lib_path(), build.kernel_sources(), build.HIP_FLAGS),
                               (build.host_lib_path(), build.host_sources(), build.HOST_FLAGS)):
        state = "current" if build.is_current(path, build.sources_digest(files, flags)) else "missing or stale: rebuilt at first use"
        lines.append(f"native library {path}: {state}")
    return lines


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """Model folders of the tiny configurations, written once per session in a temporary place."""
    import helpers

    root = tmp_path_factory.mktemp("models")
    return {name: helpers.write_model(str(root / name), name) for name in helpers.CONFIGS}
