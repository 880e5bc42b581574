"""lego_amd: LEGO layout algebra with an MI355X (gfx950) HIP lowering.

``from lego_amd import *`` gives the layout API (``OrderBy``, ``Row``, ``Col``, ``RegP``,
``GenP``, ``GroupBy``, ``TileBy`` ...), as ``import lego`` does in the reference
(lego/__init__.py:1).  The lowerings live in ``lego_amd.lego_python``, ``lego_amd.lego_c``
and ``lego_amd.lego_hip``; none of them is imported here, so importing the package
needs neither a compiler nor a GPU.
"""
from .lego import *  # noqa: F401,F403
