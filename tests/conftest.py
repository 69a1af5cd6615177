import pathlib
import sys

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


_OPTION_DEFAULTS = {"chunks": 0, "letter_bounds": 1, "logsig_scatter": 0, "batch_tile": 0, "embed_share": -1, "tiled": 1,
                    "deep_fp64": 1, "grouped": 1}


@pytest.fixture
def set_option():
    """Sets tuning switches of the kernel library for one test and restores the defaults afterwards."""
    from pathsig_amd import _load

    def setter(name, value):
        _load.set_option(name, value)

    yield setter
    for name, value in _OPTION_DEFAULTS.items():
        _load.set_option(name, value)
