import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def c_oracle():
    from oracle.c_binding import load_c_oracle

    return load_c_oracle(build_if_missing=True)


@pytest.fixture(scope="session")
def native_lib():
    """The built HIP library; built on first use only if no library exists yet."""
    import dflash_mlx_amd._native as nat

    if not nat.is_built():
        import importlib.util

        spec = importlib.util.spec_from_file_location(
            "dflash_build_ext", os.path.join(ROOT, "dflash-mlx_amd", "build_ext.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build()
    return nat.lib()


@pytest.fixture()
def verify_env(monkeypatch):
    """Environment of an enabled verify kernel with default dispatch."""
    monkeypatch.setenv("DFLASH_VERIFY_QMM", "1")
    for name in ("DFLASH_VERIFY_VARIANT", "DFLASH_VERIFY_QMM_KPARTS", "DFLASH_VERIFY_MAX_N",
                 "DFLASH_VERIFY_INCLUDE", "DFLASH_VERIFY_LINEAR", "DFLASH_REPLAY_EXACT", "DFLASH_QMM_KERNEL"):
        monkeypatch.delenv(name, raising=False)
    return monkeypatch
