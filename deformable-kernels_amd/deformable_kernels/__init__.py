"""Deformable kernels for AMD MI355X (gfx950).

Drop-in for the ``deformable_kernels`` package of hangg7/deformable-kernels:
same module names, constructor arguments, state-dict keys and tensor layouts
(reference ``deformable_kernels/modules/__init__.py:10-26``), running on
hand-written HIP kernels behind a C ABI (``include/dk_hip.h``).
"""
__version__ = "0.1.0"
