"""Host-side mirror of the reference's ``astrai.extension`` for the quantized
linear path: registry (``loader``), custom ops (``ops``), scaling policy and the
``aten::linear`` override (``fp8``, ``w8a8``)."""

from astrai_amd.extension.loader import KERNEL_NAMES, get_module, is_available

__all__ = ["KERNEL_NAMES", "get_module", "is_available"]
