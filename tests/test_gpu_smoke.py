"""The entry point the build harness runs on the GPU: one small fused step through lpmm.optim.AdamW
against the oracle (codes and scales exact, parameters within the fused kernel's bound)."""
import os
import sys

import pytest

pytestmark = pytest.mark.gpu


def test_smoke_entry_point(capsys):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    if root not in sys.path:
        sys.path.insert(0, root)
    import __graft_entry__

    __graft_entry__.smoke()
    assert "smoke ok" in capsys.readouterr().out
