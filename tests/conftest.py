import importlib.util
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TESTS = os.path.dirname(os.path.abspath(__file__))
if TESTS not in sys.path:
    sys.path.insert(0, TESTS)


def load_package():
    """Imports ncnn-moe-runtime_amd/ (not a valid identifier) under the name ncnn_moe_runtime_amd."""
    if "ncnn_moe_runtime_amd" in sys.modules:
        return sys.modules["ncnn_moe_runtime_amd"]
    package_dir = os.path.join(ROOT, "ncnn-moe-runtime_amd")
    spec = importlib.util.spec_from_file_location(
        "ncnn_moe_runtime_amd", os.path.join(package_dir, "__init__.py"),
        submodule_search_locations=[package_dir])
    module = importlib.util.module_from_spec(spec)
    sys.modules["ncnn_moe_runtime_amd"] = module
    spec.loader.exec_module(module)
    return module


load_package()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a MI355X (run on the GPU box)")
    config.addinivalue_line("markers", "reference: needs the reference library built from /root/reference")
