"""Host executor restating the reference's NumPy simulator (test
infrastructure only; see oracle/__init__.py)."""

from .executor import (Buffer, CurrentGroup, CurrentGroup1, CurrentGroup2,
                       CurrentGroup3, CurrentSubGroup, CurrentWorkitem, Kernel,
                       TunableParam, Typename, atomic_ref, kernel,
                       resolve_symbols, sym, typename)
from .tiles import Mapping, Tile, create_mapping

__all__ = ["Buffer", "CurrentGroup", "CurrentGroup1", "CurrentGroup2",
           "CurrentGroup3", "CurrentSubGroup", "CurrentWorkitem", "Kernel",
           "Mapping", "Tile", "TunableParam", "Typename", "atomic_ref",
           "create_mapping", "kernel", "resolve_symbols", "sym", "typename"]
