"""mummu_amd: the OLMoE / Qwen-MoE sparse mixture-of-experts block for MI355X (gfx950).

Hand-written HIP kernels behind the C ABI of ``include/mummu_moe.h``; this package is the thin
host-side mirror of the reference's module interface (``SparseMoe``, ``SparseMoePerExpert``,
``RoutedExperts``) over that ABI, plus seeded synthetic inputs.  Nothing here computes on the
CPU: without the built HIP library and a GPU every call raises.
"""
from . import synth  # noqa: F401

__all__ = ["synth"]
