"""MI355X (gfx950) implementation of the torkit3d point-cloud operator library.

``torkit3d_amd.ops`` mirrors ``torkit3d.ops`` of the reference (same modules,
function names, argument order, defaults and return order); ``torkit3d_amd._C``
mirrors the reference's compiled extension ``torkit3d._C``. The arithmetic lives in
hand-written HIP kernels behind the C ABI declared in ``include/tk3d.h``.
"""
__version__ = "0.1.0"
