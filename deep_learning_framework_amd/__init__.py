"""MI355X-native matrix-multiplication path of the KONAN AI engine.

The product is ``libkai_hip.so`` (hand-written HIP kernels for gfx950 behind the C-ABI of
``include/kai_hip.h``); this package holds its sources (``csrc/``), the ctypes binding
(``kai``) and a host-side mirror of the engine's tensor operators that call the path
(``tensor_ops``).  Importing the package does not load the library; ``kai.load()`` does and
raises if it has not been built.
"""
from . import kai  # noqa: F401

__all__ = ["kai", "tensor_ops"]
