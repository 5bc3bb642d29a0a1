import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


# Every device buffer the library allocates during the tests starts filled with 0xFF bytes (NaN as a float),
# and the GPU tests also overwrite the LDS of every CU with NaNs before they run: memory on a GPU keeps what
# the last user left there, so a kernel that reads what nobody wrote passes or fails by what ran before it
# unless the tests make that content hostile.
os.environ.setdefault("HOMURA_ALLOC_FILL", "0xFF")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _hostile_lds(request):
    if request.node.get_closest_marker("gpu") is not None:
        request.getfixturevalue("ctx").fill_lds()
    yield


@pytest.fixture(scope="session")
def golden():
    import json
    return json.loads((ROOT / "tests" / "golden" / "reference_vectors.json").read_text())


@pytest.fixture(scope="session")
def oracle():
    import pyoracle
    pyoracle.load()
    return pyoracle


@pytest.fixture(scope="session")
def ctx():
    """One GPU context for the whole session (GPU tests only)."""
    import homura_amd
    c = homura_amd.Context(0)
    yield c
    c.__exit__(None, None, None)
