import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (test infrastructure)."""
    from oracle import arcq_ref
    arcq_ref.build_c_oracle()
    return arcq_ref


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from arcq_vit_amd import _lib
    _lib.load()  # raises if the HIP library is not built: GPU tests must not pass without it
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _arcq_tuning_env(monkeypatch):
    """The library reads its ARCQ_* tuning variables once per process: re-read them whenever a test changes one
    through ``monkeypatch``, and once more after the test's changes have been undone."""
    import os
    from arcq_vit_amd import _lib
    touched = []

    def reload():
        if os.path.exists(_lib.LIB_PATH):
            _lib.reload_tuning()

    orig_set, orig_del = monkeypatch.setenv, monkeypatch.delenv

    def setenv(name, value, *a, **k):
        orig_set(name, value, *a, **k)
        if name.startswith("ARCQ_"):
            touched.append(name)
            reload()

    def delenv(name, *a, **k):
        orig_del(name, *a, **k)
        if name.startswith("ARCQ_"):
            touched.append(name)
            reload()

    monkeypatch.setenv, monkeypatch.delenv = setenv, delenv
    yield
    if touched:
        monkeypatch.undo()
        reload()
