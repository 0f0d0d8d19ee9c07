import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    # quantize_dynamic (the swap mechanism the reference uses too) announces its deprecation on every call
    config.addinivalue_line("filterwarnings", "ignore:torch.ao.quantization is deprecated:DeprecationWarning")


def pytest_collection_modifyitems(config, items):
    # Every GPU test announces itself (flushed) before it touches the device, so a
    # run that loses the box still names the case that was executing.
    pass


@pytest.fixture(autouse=True)
def _announce(request):
    if request.node.get_closest_marker("gpu") is not None:
        print(f"\n[gpu-case] {request.node.nodeid}", flush=True)
    yield


@pytest.fixture
def tuning():
    """Setter of the library's tuning overrides (tra_set_tuning); every knob goes
    back to its default when the test ends."""
    from torchrec_amd import _lib

    touched = set()

    def set_(**knobs):
        touched.update(knobs)
        _lib.set_tuning(**knobs)

    yield set_
    if touched:
        _lib.set_tuning(**{k: None for k in touched})
