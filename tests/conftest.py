import json
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (ROOT, ROOT / "oracle"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def exact_cases():
    """Exact-rational problems and their exact derivatives (tests/golden/make_exact_vectors.py)."""
    data = json.loads((ROOT / "tests" / "golden" / "fm_scan_exact.json").read_text())
    return {c["name"]: c for c in data["cases"]}
