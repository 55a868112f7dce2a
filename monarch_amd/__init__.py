"""monarch_amd: MI355X-native data plane for Monarch's mesh data-movement / reduce path.

Host-side mirror of the reference's interfaces for this path (``Slice``, ``DeviceMesh``,
``RDMABuffer`` staging, ``Reduce``) over the C ABI of ``libmonarch_hip.so``.  Importing the
package does not load the library; the first call does, and fails loudly if it was not built.
"""
from ._lib import LIB_PATH, MhipError, MonarchHipNotBuilt, lib  # noqa: F401
from .ndslice import Slice  # noqa: F401
from .device_mesh import DeviceMesh, Dim  # noqa: F401

__all__ = ["Slice", "DeviceMesh", "Dim", "MhipError", "MonarchHipNotBuilt", "lib", "LIB_PATH"]
