"""The driver's smoke entry point, run as part of the GPU suite so that it cannot rot."""
import os
import sys

import pytest

pytestmark = pytest.mark.gpu

pytest.importorskip("torch")


def test_graft_entry_smoke():
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import __graft_entry__ as entry

    entry.smoke()
