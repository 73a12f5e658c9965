import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """A gpu test that finds no GPU fails loudly rather than being skipped in
    silence, unless -m selects it away."""
    return


@pytest.fixture(scope="session")
def tiny_configs():
    from kipp_amd.config import shape_config
    return {"a": shape_config("tiny-a"), "b": shape_config("tiny-b")}


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory, tiny_configs):
    """Random-weight model folders of both tiny configurations, in float32 and
    in bfloat16, made in a temporary folder."""
    from kipp_amd.weights import write_random_model
    root = tmp_path_factory.mktemp("models")
    out = {}
    for key, cfg in tiny_configs.items():
        for dtype in ("float32", "bfloat16"):
            out[(key, dtype)] = write_random_model(str(root / f"tiny-{key}-{dtype}"), cfg, seed=1234 + ord(key), dtype=dtype)
    return out
