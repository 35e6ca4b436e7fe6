"""Shared pytest configuration: the `gpu` marker and import paths.

Tests marked `gpu` need a real MI355X and go through the C-ABI library; everything else
runs on CPU (oracle pinning, host-side argument checks, symbol export checks).
"""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "strassen-triton_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (runs through the HIP C-ABI library)")


def _has_gpu() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def force_tile():
    """force_tile("256x256") overrides the library's tile table (sthip_debug_force_tile) until the
    test ends; the previous setting comes back afterwards."""
    from strassen_hip import _capi
    lib = _capi.load()
    names = {0: None, 2: b"128x128", 3: b"256x128", 4: b"256x256", 5: b"128x128g", 6: b"64x64"}
    first = []

    def force(tile):
        prev = lib.sthip_debug_force_tile(tile.encode() if tile else None)
        if not first:
            first.append(prev)

    yield force
    if first:
        lib.sthip_debug_force_tile(names[first[0]])


@pytest.fixture(scope="session")
def host_builds(tmp_path_factory):
    """The kernels and the library compiled for the host (tests/test_kernel_host_model.py says how): host_builds("asan") etc."""
    from test_kernel_host_model import HostBuilds
    return HostBuilds(str(tmp_path_factory.mktemp("host_model")))
