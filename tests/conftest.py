import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) device")


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from merak_amd import _lib
    _lib.lib()  # raises if the kernel library has not been built: never silently fall back
    assert _lib.device_arch() == "gfx950"
    return torch.device("cuda:0")


@pytest.fixture
def set_tuning(monkeypatch):
    """set_tuning(name, value): put an MTP_* tuning variable into the environment (None removes it) and have the
    library read it: the library reads its environment once, not per launch.  Undone when the test ends."""
    from merak_amd import _lib

    def _set(name, value):
        if value is None:
            monkeypatch.delenv(name, raising=False)
        else:
            monkeypatch.setenv(name, str(value))
        _lib.lib().mtp_reload_tuning()

    yield _set
    monkeypatch.undo()
    _lib.lib().mtp_reload_tuning()


@pytest.fixture(autouse=True)
def _reset_mpu():
    from merak_amd import mpu, set_args
    mpu.destroy_model_parallel()
    mpu.get_rng_tracker().reset()
    set_args(use_cpu_initialization=True)
    yield
    mpu.destroy_model_parallel()
    mpu.get_rng_tracker().reset()
