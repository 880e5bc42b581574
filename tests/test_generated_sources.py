"""The tracked sources under lego_amd/csrc/generated/ are what the generators emit: every file, byte for
byte, and no file that no generator owns (they are build output kept in the tree so that the kernels
can be read without running sympy)."""
from lego_amd import build
from lego_amd.kernels.common import GENERATED


def test_generators_reproduce_the_tracked_sources():
    units, header = build.collect()
    assert (GENERATED / "launchers.h").read_text() == header
    names = set()
    for unit in units:
        assert (GENERATED / unit.filename).read_text() == unit.text, unit.filename
        names.add(unit.filename)
    assert len(names) == len(units)                                   # no two units share a file
    assert {p.name for p in GENERATED.glob("*.hip")} == names         # and nothing else lies there
