import os
import sys
from pathlib import Path

import pytest

# The library honours its MOGRAD_HIP_* tuning knobs only in a process that opts in; the
# equivalence tests flip kernel layouts through them.  It reads the switch once, so set it
# before the library is loaded.
os.environ.setdefault("MOGRAD_HIP_TUNING", "1")

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def device():
    """One Device for the whole session: a single GPU process, a single stream."""
    from mograd_amd import Device

    dev = Device()
    yield dev
    dev.synchronize()
