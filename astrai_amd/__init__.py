"""astrai_amd: gfx950 (MI355X) backend for AstrAI's quantized linear-layer GEMM path.

Only the hot path lives here: HIP kernels and their C ABI (``csrc/``), and the
host-side mirror of the reference's ``astrai/extension`` interface for that path
(``extension/``: kernel registry, custom ops, scaling policy, ``aten::linear``
override).
"""

__version__ = "0.1.0"
