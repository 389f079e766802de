import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture
def opts():
    """``opts(field=value, ...)``: sets ``mmsim_options`` fields on the default context for the rest of the
    test (on top of what the test set before); the defaults come back afterwards."""
    from mms_amd import engine as E
    touched = []

    def set_fields(**fields):
        eng = E.Engine.default()
        eng.set_options(**{**getattr(eng, "_options", {}), **fields})
        touched.append(eng)
    yield set_fields
    for eng in touched:
        eng.set_options()


@pytest.fixture(params=["oracle", pytest.param("gpu", marks=pytest.mark.gpu)])
def backend(request, monkeypatch):
    """Host logic runs twice: with the CPU oracle standing in for the library, and (marked gpu) through libmmsim."""
    if request.param == "oracle":
        import oracle_backend
        oracle_backend.install(monkeypatch)
    return request.param
