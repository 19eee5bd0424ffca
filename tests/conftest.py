import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# the reference checkout's own fixture; SPROUT_REFERENCE_FIXTURE names a copy where the checkout is not mounted
REFERENCE_FIXTURE = os.environ.get("SPROUT_REFERENCE_FIXTURE", "/root/reference/test/fixtures/qwen-tiny")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X and the built HIP library")


@pytest.fixture(scope="session")
def reference_fixture():
    """The reference's own tiny Qwen2 with logits computed by an independent library.

    Read in place (never copied); tests that need it are skipped where the
    reference checkout is not mounted.
    """
    if not os.path.isfile(os.path.join(REFERENCE_FIXTURE, "reference.json")):
        pytest.skip("reference fixture not mounted")
    return REFERENCE_FIXTURE
