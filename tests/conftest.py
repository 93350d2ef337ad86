import sys
from pathlib import Path

import pytest

import os
import tempfile

ROOT = Path(__file__).resolve().parents[1]
# generated code objects are cached per user under $XDG_CACHE_HOME; the tests keep theirs out of the home directory
os.environ.setdefault("XDG_CACHE_HOME", str(Path(tempfile.gettempdir()) / f"ilang_test_cache_{os.getuid()}"))
Path(os.environ["XDG_CACHE_HOME"]).mkdir(mode=0o700, exist_ok=True)
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import numpy as np

    return np.load(ROOT / "tests" / "golden" / "flashattn_ref.npz")
