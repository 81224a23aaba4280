import ctypes
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X); skipped by -m 'not gpu'")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no HIP device in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle_c():
    """The plain-C oracle (oracle/oracle_c.c), built on demand with gcc."""
    from oracle import build as obuild

    path = obuild.OUT
    src = path.parent.parent / "oracle_c.c"
    if not path.exists() or path.stat().st_mtime < src.stat().st_mtime:
        obuild.build(verbose=False)
    lib = ctypes.CDLL(str(path))
    i64, vp, ci, cf = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    lib.orc_reduce.argtypes = [vp, ci, i64, i64, vp, i64, ci, vp]
    lib.orc_reduce.restype = None
    lib.orc_reduce_rmsnorm.argtypes = [vp, ci, i64, i64, i64, vp, ci, vp, cf, vp, vp]
    lib.orc_reduce_rmsnorm.restype = None
    lib.orc_gemm.argtypes = [vp, vp, i64, i64, i64, vp, ci, vp, vp]
    lib.orc_gemm.restype = None
    return lib


@pytest.fixture(scope="session")
def dev():
    return torch.device("cuda:0")


class _EnvAwareMonkeyPatch:
    """pytest's monkeypatch, except that a change to a KRAKEN_AMD_* variable also makes the
    library read its switches again (it reads the environment once per process)."""

    def __init__(self, inner):
        self._inner = inner

    def __getattr__(self, name):
        return getattr(self._inner, name)

    @staticmethod
    def _reload(name):
        if name.startswith("KRAKEN_AMD_"):
            from kraken_amd import _lib

            _lib.reload_env()

    def setenv(self, name, value, prepend=None):
        self._inner.setenv(name, value, prepend)
        self._reload(name)

    def delenv(self, name, raising=True):
        self._inner.delenv(name, raising)
        self._reload(name)


@pytest.fixture
def monkeypatch(monkeypatch):
    yield _EnvAwareMonkeyPatch(monkeypatch)
    monkeypatch.undo()
    from kraken_amd import _lib

    _lib.reload_env()
