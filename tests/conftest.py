import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as orc

    orc.lib()
    return orc


@pytest.fixture(scope="session")
def golden_dir():
    return GOLDEN


@pytest.fixture(autouse=True)
def _tuning_follows_environment(monkeypatch):
    """The library reads its FOS_* overrides once; tests that set them go through this hook,
    and every test starts from the environment as it is."""
    from fouroversix_amd import _native as nat

    if not os.path.exists(nat.LIB_PATH):
        yield
        return
    reload_tuning = nat.lib().fos_tuning_reload
    reload_tuning()
    set_env, del_env = monkeypatch.setenv, monkeypatch.delenv

    def setenv(name, value, *a, **kw):
        set_env(name, value, *a, **kw)
        reload_tuning()

    def delenv(name, *a, **kw):
        del_env(name, *a, **kw)
        reload_tuning()

    monkeypatch.setattr(monkeypatch, "setenv", setenv, raising=False)
    monkeypatch.setattr(monkeypatch, "delenv", delenv, raising=False)
    yield
