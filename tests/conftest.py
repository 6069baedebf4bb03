import importlib.util
import json
import pathlib
import sys

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    with open(ROOT / "tests" / "golden" / "reference_test_vectors.json") as f:
        return json.load(f)


@pytest.fixture(scope="session")
def ref_C():
    """The reference's own util.cpp, compiled by oracle/Makefile into
    oracle/_ref (absent when that build was not run)."""
    hits = sorted((ROOT / "oracle" / "_ref").glob("_C*.so"))
    if not hits:
        pytest.skip("oracle/_ref/_C not built (run make -C oracle)")
    import torch  # noqa: F401  (the extension links against libtorch)

    spec = importlib.util.spec_from_file_location("_C", hits[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def pbg():
    """The shipped package (directory pytorch-biggraph_amd, imported as
    pytorch_biggraph_amd)."""
    import __graft_entry__

    return __graft_entry__.load_package()
