"""raven_amd — an MI355X (gfx950) engine behind Nx's backend contract.

The package holds the HIP kernel library with its C ABI (``csrc/``, built into
``libnxhip.so``), and a Python mirror of the OCaml binding that sits on top of
that ABI (``nx_backend``), with the same operation names, argument meaning and
error kinds as ``Nx_core.Backend_intf.S`` (raven-ml/raven,
packages/nx/lib/core/backend_intf.ml:77-721).
"""

from . import dtype, view  # noqa: F401

__all__ = ["dtype", "view"]
