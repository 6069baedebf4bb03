"""The driver's smoke entry point runs as part of the GPU suite."""
import pytest


@pytest.mark.gpu
def test_smoke_entry_point():
    import __graft_entry__

    __graft_entry__.smoke()
