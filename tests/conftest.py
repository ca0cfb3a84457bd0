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


@pytest.fixture(autouse=True)
def decode_graphs_from_the_first_step(monkeypatch):
    """The engine captures a decode step's graph the third time its shape comes and runs it
    eagerly before that; tests decode only a few steps, so here every shape is captured at once
    and the graph path is what they check.  ``test_a_shape_is_captured_the_third_time_it_comes``
    sets the engine's own value back."""
    from from_scratch_inference_engine_amd.engine import graphs

    monkeypatch.setattr(graphs, "CAPTURE_AFTER", 1)
