import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X); run with -m gpu")


import os

import pytest


@pytest.fixture
def tune():
    """Sets / clears BP_TUNE_* development switches and makes the library read them again (it reads them once when it
    is first used); the environment and the library's copy are restored afterwards."""
    from deepseekternarized_amd.kernels import _lib

    saved = {}

    def set_(name, value):
        saved.setdefault(name, os.environ.get(name))
        if value is None:
            os.environ.pop(name, None)
        else:
            os.environ[name] = value
        _lib.load().bp_reload_tuning()

    yield set_
    for name, old in saved.items():
        if old is None:
            os.environ.pop(name, None)
        else:
            os.environ[name] = old
    _lib.load().bp_reload_tuning()
