import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def _ensure_built():
    """The tests load what is built; only a tree where nothing has been built yet gets a build
    (hipcc cross-compiles gfx950 without a GPU; the oracle needs gcc)."""
    lib = ROOT / "triton-tenstorrent_amd" / "lib" / "libttamd_rt.so"
    orc = ROOT / "oracle" / "liboracle.so"
    if lib.exists() and orc.exists():
        return
    import importlib
    entry = importlib.import_module("__graft_entry__")
    entry.build()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    _ensure_built()


def _has_gpu() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
