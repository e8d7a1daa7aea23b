"""MI355X-native execution backend for PET tensor programs.

``pet_amd.abi`` binds the C-ABI shared library (``include/pet_hip.h``),
``pet_amd.ops`` calls it on torch device tensors. All compute happens in the
HIP library; importing this package never falls back to a CPU path.
"""
from . import abi  # noqa: F401

__all__ = ["abi"]
