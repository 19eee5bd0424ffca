import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# test vectors that the reference's own tests hold: the copy kept beside the tests, or the folder that
# SPROUT_REFERENCE_FIXTURE names
REFERENCE_FIXTURE = os.environ.get("SPROUT_REFERENCE_FIXTURE") or os.path.join(ROOT, "tests", "fixtures", "reference_qwen_tiny")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X and the built HIP library")


@pytest.fixture(scope="session")
def reference_fixture():
    """The reference's own tiny Qwen2 with logits computed by an independent library.

    Tests that need it are skipped where the folder is not there.
    """
    if not os.path.isfile(os.path.join(REFERENCE_FIXTURE, "reference.json")):
        pytest.skip(f"no reference fixture at {REFERENCE_FIXTURE}")
    return REFERENCE_FIXTURE
