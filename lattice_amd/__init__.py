"""MI355X-native Q4 block-quantized matmul path for lattice (gfx950 / CDNA4).

Public surface: :mod:`lattice_amd.backend` (host-side mirror of the reference's
``dispatch_matmul`` / ``dispatch_gemm`` / ``dispatch_lora_if_active`` contract over the
C ABI in ``include/lattice_hip_q4.h``), :mod:`lattice_amd.q4_layout` (the 20-byte block
layout) and :mod:`lattice_amd.synth` (seeded synthetic workloads).
"""
__all__ = ["q4_layout", "synth"]
