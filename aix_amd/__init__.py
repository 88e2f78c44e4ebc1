"""aix_amd -- an MI355X (gfx950) device backend for the AIX operator interface.

Two shared libraries live next to this file once built (``aix_amd.build()``):

* ``libaixhip_kernels.so`` -- hand-written HIP kernels behind a thin C ABI
  (``include/aixhip_kernels.h``), bound in :mod:`aix_amd.kernels`;
* ``libaixhip.so`` -- the lazy, fusing ``DeviceHIP`` (C++) behind a C ABI that mirrors
  ``aix::Device`` method for method (``include/aixhip.h``), bound in :mod:`aix_amd.device`.

There is no CPU fallback anywhere in this package: if a library is missing or no GPU is
visible, calls raise.
"""
from ._build import build, library_path  # noqa: F401
