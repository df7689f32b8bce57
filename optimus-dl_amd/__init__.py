"""MI355X-native FP8 AMP Linear path for Optimus-DL.

Importable as ``optimus_dl_amd``.  Layout mirrors the part of the reference tree
that this path touches (``core``, ``modules.amp``, ``modules.optim``,
``modules.model_transforms``, ``modules.model``), plus ``csrc`` (HIP kernels and
the C ABI), ``native`` (ctypes binding) and ``build`` (hipcc recipe).
"""

__version__ = "0.1.0"
