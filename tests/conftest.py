import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run on the GPU box with -m gpu)")


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders of the two tiny configurations, weights stored as bfloat16 so that the
    float32 and the bfloat16 runs and the plain implementation all read the same values."""
    import helpers

    root = tmp_path_factory.mktemp("models")
    return {name: helpers.make_model_dir(root / name, cfg, seed)
            for name, (cfg, seed) in helpers.TINY.items()}
