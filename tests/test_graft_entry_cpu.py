"""__graft_entry__.smoke() -- the small invocation of the hot path the driver runs on a GPU -- run against the CPU build
of the library (tests/emu_util.py), so that what it asks for (kernel names, shapes, the oracle comparisons) is known to
hold before a GPU sees it."""
import os
import sys

import pytest

import emu_util
from hodu_amd import ffi

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
pytestmark = pytest.mark.skipif(emu_util.compiler() is None, reason="no host clang++ for the CPU build")


def test_smoke_passes_in_the_cpu_build(monkeypatch, capsys):
    import __graft_entry__ as entry
    monkeypatch.setattr(ffi, "Context", emu_util.EmuContext)
    entry.smoke()
    assert "smoke ok" in capsys.readouterr().out
