"""MI355X-native MoE expert-layer forward (the SparseMoE path of Jaxtitan).

``research_amd.moe`` mirrors the reference layer's interface, ``research_amd.ops``
exposes the stage operators, ``research_amd._ffi`` binds the C ABI of
``include/jtmoe.h`` and ``research_amd.build`` compiles it.  Nothing here has a
CPU or eager fallback: without the built HIP library every operator raises.
"""

__all__ = ["build", "errors", "moe", "ops"]
